"""The operator class end to end on the GPU: heuristic_prepare -> workspace ->
forward() (append, decode, chunked prefill on one stream), checked against the
CPU oracle: cache bytes and scales bit-exact, outputs within tolerance."""
import numpy as np
import pytest
import torch

from conftest import (assert_attention_close, host_cache, oracle_append_step, oracle_decode, oracle_fill_history,
                      oracle_prefill)

pytestmark = pytest.mark.gpu


def full_step(pkg, oracle, bt, rng, **op_kw):
    cache, scale = host_cache(bt, canary=(0x5A, 1.5))
    dev = pkg.harness.DeviceBatch(bt)
    dev.fill_canary()
    for b, pos, k_rows, v_rows in oracle_fill_history(oracle, pkg, bt, rng, cache, scale):
        dev.append_rows(b, pos, k_rows, v_rows)
    q, k, v = pkg.workloads.step_inputs(bt, rng)
    dev.set_step_inputs(q, k, v)
    dev.output.fill_(float("nan"))
    op = dev.make_operator(**op_kw)
    rc = op.forward()
    torch.cuda.synchronize()
    assert rc == 0
    oracle_append_step(oracle, bt, k, v, cache, scale)
    assert np.array_equal(dev.cache.cpu().numpy(), cache)
    assert np.array_equal(dev.scale.cpu().numpy().view(np.uint16), scale.view(np.uint16))
    ref = oracle_prefill(oracle, bt, q, cache, scale) if bt.batch > bt.decoding_batches else np.zeros(
        (q.shape[0], bt.num_heads, bt.head_dim), np.float32)
    if bt.decoding_batches:
        ref[:bt.decoding_batches] = oracle_decode(oracle, bt, q, cache, scale)
    got = dev.output.float().cpu().numpy()
    return assert_attention_close(got, ref, bt.name), op


def test_c1_through_the_operator(pkg, oracle):
    bt, rng = pkg.workloads.make_batch("C1")
    full_step(pkg, oracle, bt, rng)


@pytest.mark.parametrize("multi_block", [0, 1, 2])
def test_mixed_batch_through_the_operator(pkg, oracle, multi_block):
    bt, rng = pkg.workloads.custom_batch(401, num_heads=32, num_kv_heads=8, head_dim=128, cache_mode=1,
                                         dec_kv_lens=[600, 33, 1500, 129, 1, 256], prefill_q_lens=[100, 17],
                                         prefill_prior=[150, 0], outliers=True, num_layer=2, layer_idx=1)
    _, op = full_step(pkg, oracle, bt, rng, specify_decoding_multi_block=multi_block)
    if multi_block == 0:
        assert op.cfg.decoding_multi_block_size == 1 and op.cfg.workspace_size == 0


@pytest.mark.parametrize("heads", [(16, 8, 256), (8, 8, 256), (12, 4, 96), (32, 4, 256)])
def test_mixed_batch_at_the_other_head_dims(pkg, oracle, heads):
    """head_dim 96 and 256 (the reference's flash attention and decode kernels serve 64, 96, 128, 256): append,
    decode and the 16-column prefill kernel in one forward()."""
    hq, hkv, d = heads
    bt, rng = pkg.workloads.custom_batch(420 + hq + d, num_heads=hq, num_kv_heads=hkv, head_dim=d, cache_mode=1,
                                         dec_kv_lens=[300, 33, 700, 1], prefill_q_lens=[100, 17, 130],
                                         prefill_prior=[150, 0, 31], outliers=True, num_layer=2, layer_idx=1)
    full_step(pkg, oracle, bt, rng)


@pytest.mark.parametrize("heads,q_lens", [((32, 8, 128), [4, 8, 1, 5]), ((8, 8, 64), [32, 2, 17, 9]), ((16, 2, 128), [3, 4, 2, 1]),
                                          ((32, 8, 128), [4, 2, 1, 3])])
def test_mixed_batch_with_short_chunks(pkg, oracle, heads, q_lens):
    """Decode sequences plus chunks of a few query tokens (speculative decoding's candidates): the operator's workspace
    covers the prefill stage's pieces too, and forward() runs those chunks on the decode step's kernel."""
    hq, hkv, d = heads
    bt, rng = pkg.workloads.custom_batch(430 + hq + d, num_heads=hq, num_kv_heads=hkv, head_dim=d, cache_mode=1,
                                         dec_kv_lens=[300, 33, 1700, 1], prefill_q_lens=q_lens,
                                         prefill_prior=[1500, 0, 640, 2047], outliers=True, num_layer=2, layer_idx=1)
    assert pkg.ops.prefill_workspace_size(bt.batch, bt.decoding_batches, bt.max_seqlen, bt.max_kvlen, hq, hkv, d) > 0
    full_step(pkg, oracle, bt, rng)


def test_scaled_c5_through_the_operator(pkg, oracle):
    bt, rng = pkg.workloads.make_batch("C5", scale=0.06)
    full_step(pkg, oracle, bt, rng)


@pytest.mark.parametrize("heads", [(32, 8, 128), (64, 8, 128), (8, 8, 64)])
def test_cache_beyond_4_gib(pkg, oracle, heads):
    """A cache of many layers whose last layer lies more than 4 GiB into the allocation (a serving cache on a
    288 GB part is tens of GiB): every kernel's element offsets must be 64-bit.  The whole cache is compared, so
    a write at a wrapped offset shows as a damaged canary in another layer."""
    hq, hkv, d = heads
    kw = dict(num_heads=hq, num_kv_heads=hkv, head_dim=d, cache_mode=1, dec_kv_lens=[600, 33, 1500, 129, 1, 256],
              prefill_q_lens=[100, 17], prefill_prior=[150, 0], outliers=True)
    probe, _ = pkg.workloads.custom_batch(405, num_layer=1, layer_idx=0, **kw)
    layer_bytes = 2 * probe.layout.pool_tokens * hkv * d
    layers = (4 << 30) // layer_bytes + 3
    bt, rng = pkg.workloads.custom_batch(405, num_layer=layers, layer_idx=layers - 1, **kw)
    assert bt.layer_idx * layer_bytes > (4 << 30)
    full_step(pkg, oracle, bt, rng)


@pytest.mark.parametrize("q_lens,prior", [([70], [300]), ([4, 7, 1], [1300, 40, 2000])])
def test_forward_in_a_hip_graph(pkg, oracle, q_lens, prior):
    """forward() records no memory-set node and allocates nothing, so a caller can capture it: every replay,
    with eager calls between the replays, gives the rows of the eager call bit for bit.  With a prefill chunk on the
    tile kernel, and with short chunks on the decode step's kernel."""
    bt, rng = pkg.workloads.custom_batch(404, num_heads=32, num_kv_heads=8, head_dim=128, cache_mode=1,
                                         dec_kv_lens=[700, 2, 1900, 130, 1], prefill_q_lens=q_lens, prefill_prior=prior,
                                         outliers=True)
    cache, scale = host_cache(bt)
    dev = pkg.harness.DeviceBatch(bt)
    for b, pos, k_rows, v_rows in oracle_fill_history(oracle, pkg, bt, rng, cache, scale):
        dev.append_rows(b, pos, k_rows, v_rows)
    q, k, v = pkg.workloads.step_inputs(bt, rng)
    dev.set_step_inputs(q, k, v)
    op = dev.make_operator(specify_decoding_multi_block=1)
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        assert op.forward(side) == 0  # also sets the kernels' attributes before the capture
        side.synchronize()
        eager = dev.output.clone()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            assert op.forward(side) == 0
            assert op.forward(side) == 0
        for rep in range(3):
            dev.output.fill_(float("nan"))
            graph.replay()
            side.synchronize()
            assert torch.equal(dev.output.view(torch.int16), eager.view(torch.int16)), "replay %d" % rep
            assert op.forward(side) == 0
            side.synchronize()
    oracle_append_step(oracle, bt, k, v, cache, scale)
    ref = oracle_prefill(oracle, bt, q, cache, scale)
    ref[:bt.decoding_batches] = oracle_decode(oracle, bt, q, cache, scale)
    assert_attention_close(eager.float().cpu().numpy(), ref, "eager rows")


@pytest.mark.parametrize("q_lens,prior", [([70, 300], [300, 0]), ([4, 7, 1], [1300, 40, 2000])])
def test_forward_on_two_streams(pkg, oracle, q_lens, prior):
    """forward(stream, side_stream, fork, join): the decode stage beside the prefill stage.  Same kernels on the same
    inputs as forward(stream), so the rows are equal bit for bit -- launched from the host and replayed from a HIP
    graph captured from the main stream -- and the step is ordered before later work on the main stream.  The batch
    of short chunks shares its workspace between the stages and runs in one stream order."""
    bt, rng = pkg.workloads.custom_batch(406, num_heads=32, num_kv_heads=8, head_dim=128, cache_mode=1,
                                         dec_kv_lens=[700, 2, 1900, 130, 1, 3000], prefill_q_lens=q_lens, prefill_prior=prior,
                                         outliers=True)
    cache, scale = host_cache(bt)
    dev = pkg.harness.DeviceBatch(bt)
    for b, pos, k_rows, v_rows in oracle_fill_history(oracle, pkg, bt, rng, cache, scale):
        dev.append_rows(b, pos, k_rows, v_rows)
    q, k, v = pkg.workloads.step_inputs(bt, rng)
    dev.set_step_inputs(q, k, v)
    op = dev.make_operator(specify_decoding_multi_block=1)
    main, side = torch.cuda.Stream(), torch.cuda.Stream()
    fork, join = torch.cuda.Event(), torch.cuda.Event()
    fork.record(main)
    join.record(main)
    main.synchronize()
    with torch.cuda.stream(main):
        assert op.forward(main) == 0
        main.synchronize()
        one_stream = dev.output.clone()
        dev.output.fill_(float("nan"))
        assert op.forward_streams(main, side, fork, join) == 0
        after = dev.output.clone()  # ordered behind the join on the main stream
        main.synchronize()
        assert torch.equal(after.view(torch.int16), one_stream.view(torch.int16))
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=main):
            assert op.forward_streams(main, side, fork, join) == 0
            assert op.forward_streams(main, side, fork, join) == 0
        for rep in range(3):
            dev.output.fill_(float("nan"))
            graph.replay()
            main.synchronize()
            assert torch.equal(dev.output.view(torch.int16), one_stream.view(torch.int16)), "replay %d" % rep
    oracle_append_step(oracle, bt, k, v, cache, scale)
    ref = oracle_prefill(oracle, bt, q, cache, scale)
    ref[:bt.decoding_batches] = oracle_decode(oracle, bt, q, cache, scale)
    assert_attention_close(one_stream.float().cpu().numpy(), ref, "rows")


def test_first_step_under_capture():
    """In a fresh process: a first forward() under stream capture is refused with a message that names
    pmxhip_init(), and after that call the capture succeeds (tests/capture_first_child.py)."""
    import os
    import subprocess
    import sys
    child = os.path.join(os.path.dirname(os.path.abspath(__file__)), "capture_first_child.py")
    r = subprocess.run([sys.executable, "-u", child], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0 and r.stdout.strip().endswith("OK"), r.stdout[-2000:] + r.stderr[-2000:]


def test_contiguous_mode_and_stagewise_calls(pkg, oracle):
    bt, rng = pkg.workloads.custom_batch(402, num_heads=8, num_kv_heads=8, head_dim=64, cache_mode=0,
                                         dec_kv_lens=[200, 31], prefill_q_lens=[40], prefill_prior=[9])
    cache, scale = host_cache(bt)
    dev = pkg.harness.DeviceBatch(bt)
    for b, pos, k_rows, v_rows in oracle_fill_history(oracle, pkg, bt, rng, cache, scale):
        dev.append_rows(b, pos, k_rows, v_rows)
    q, k, v = pkg.workloads.step_inputs(bt, rng)
    dev.set_step_inputs(q, k, v)
    op = dev.make_operator()
    assert op.forward_kvstore() == 0 and op.forward_decode() == 0 and op.forward_prefill() == 0
    torch.cuda.synchronize()
    oracle_append_step(oracle, bt, k, v, cache, scale)
    ref = oracle_prefill(oracle, bt, q, cache, scale)
    ref[:2] = oracle_decode(oracle, bt, q, cache, scale)
    assert_attention_close(dev.output.float().cpu().numpy(), ref, "stagewise")


def test_unsupported_configurations_report_not_crash(pkg):
    bt, rng = pkg.workloads.custom_batch(403, num_heads=4, num_kv_heads=2, head_dim=128, cache_mode=1,
                                         dec_kv_lens=[20], prefill_q_lens=[8], prefill_prior=[0])
    dev = pkg.harness.DeviceBatch(bt)
    q, k, v = pkg.workloads.step_inputs(bt, rng)
    dev.set_step_inputs(q, k, v)
    op = dev.make_operator(datatype=6)                  # fp32 tensors: prefill rejects (flash_attn2/fmha.cu:75)
    assert op.forward_prefill() == pkg.ops.RC_UNSUPPORTED
    assert op.forward() == pkg.ops.RC_UNSUPPORTED       # first failure wins
    torch.cuda.synchronize()
