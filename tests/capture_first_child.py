"""Child process of test_gpu_operator.py::test_first_step_under_capture: a fresh process whose FIRST forward() is
recorded under stream capture.  The kernels with large dynamic LDS need one attribute call before their first
launch; under capture the library refuses (PMXHIP_OTHER_ERROR) instead of making that call inside the capture,
and after pmxhip_init() the same capture succeeds and replays the eager result.  Prints OK on success."""
import os
import sys

import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
import __graft_entry__ as entry  # noqa: E402


def main():
    pkg = entry.load_package()
    torch.cuda.set_device(0)
    bt, rng = pkg.workloads.custom_batch(406, num_heads=8, num_kv_heads=8, head_dim=64, cache_mode=1,
                                         dec_kv_lens=[700, 2, 130], prefill_q_lens=[70], prefill_prior=[300])
    dev = pkg.harness.DeviceBatch(bt)
    dev.fill_history_random_bytes(seed=1)
    q, k, v = pkg.workloads.step_inputs(bt, rng)
    dev.set_step_inputs(q, k, v)
    op = dev.make_operator(specify_decoding_multi_block=1)
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            rc = op.forward(side)
        assert rc == pkg.ops.RC_OTHER_ERROR, "first forward() under capture returned %d" % rc
        assert "pmxhip_init" in pkg._lib.last_error(), pkg._lib.last_error()
        del graph
        pkg.ops.init()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            rc = op.forward(side)
        assert rc == 0, "forward() under capture after init returned %d: %s" % (rc, pkg._lib.last_error())
        dev.output.fill_(float("nan"))
        graph.replay()
        side.synchronize()
        replayed = dev.output.clone()
        assert op.forward(side) == 0
        side.synchronize()
        assert not torch.isnan(replayed).any()
        assert torch.equal(replayed.view(torch.int16), dev.output.view(torch.int16))
    print("OK")


if __name__ == "__main__":
    main()
