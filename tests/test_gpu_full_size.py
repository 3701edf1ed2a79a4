"""Full benchmark sizes on the GPU, every output row against the CPU oracle.

The cache of each configuration is filled by the HIP quantise/append kernel from
seeded fp16 rows; for C3 and C5 the same rows also go through the oracle's
quantiser on the host and the whole cache is compared byte for byte.  One layer
call (append + decode + chunked prefill) then runs through the operator and
every output element is checked: |got - ref| <= 2e-3 + 1e-2 * |ref|."""
import numpy as np
import pytest
import torch

from conftest import (assert_attention_close, host_cache, oracle_append_step, oracle_decode, oracle_fill_history,
                      oracle_prefill)

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("name,check_whole_cache", [("C2", False), ("C3", True), ("C3m0", False), ("C4", False), ("C5", True)])
def test_full_size_layer_call(pkg, oracle, name, check_whole_cache):
    wl = pkg.workloads
    bt, rng = wl.make_batch(name)
    dev = pkg.harness.DeviceBatch(bt)
    if check_whole_cache:
        cache, scale = host_cache(bt)
        for b, pos, k_rows, v_rows in oracle_fill_history(oracle, pkg, bt, rng, cache, scale,
                                                          chunks=wl.history_chunks(bt, rng, 1 << 15)):
            dev.append_rows(b, pos, k_rows, v_rows)
        torch.cuda.synchronize()
        assert np.array_equal(dev.cache.cpu().numpy(), cache)
        assert np.array_equal(dev.scale.cpu().numpy().view(np.uint16), scale.view(np.uint16))
    else:
        dev.fill_history(rng, max_rows=1 << 15)
        cache = dev.cache.cpu().numpy()
        scale = dev.scale.cpu().numpy()
    q, k, v = wl.step_inputs(bt, rng)
    dev.set_step_inputs(q, k, v)
    dev.output.fill_(float("nan"))
    op = dev.make_operator()
    assert op.cfg.decoding_multi_block_size > 1
    assert op.forward() == 0
    torch.cuda.synchronize()
    # the rows appended by this step, bit-exact
    oracle_append_step(oracle, bt, k, v, cache, scale)
    assert np.array_equal(dev.cache.cpu().numpy(), cache)
    assert np.array_equal(dev.scale.cpu().numpy().view(np.uint16), scale.view(np.uint16))
    # every output element
    ref = (oracle_prefill(oracle, bt, q, cache, scale) if bt.batch > bt.decoding_batches
           else np.zeros((q.shape[0], bt.num_heads, bt.head_dim), np.float32))
    ref[:bt.decoding_batches] = oracle_decode(oracle, bt, q, cache, scale)
    got = dev.output.float().cpu().numpy()
    assert not np.isnan(got).any()
    assert_attention_close(got, ref, name)
    # split invariance: one token range instead of hundreds gives the same rows within rounding
    if bt.batch == bt.decoding_batches:
        few = torch.zeros_like(dev.output)
        dev.decode_only(num_token_ranges=3, output=few)
        torch.cuda.synchronize()
        assert_attention_close(few.float().cpu().numpy(), ref, name + " (3 ranges)")
