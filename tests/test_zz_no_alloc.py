"""The decode entry point that allocates nothing (pmxhip_decode_attention_static): its split-KV pieces go to a
static array inside the library instead of a caller's workspace.  Checked through the C ABI against
pmxhip_decode_attention on the same inputs, on two calls in a row, the second with a smaller input (the array
then still holds the first call's pieces)."""
import ctypes

import numpy as np
import pytest
import torch

from conftest import assert_attention_close, oracle_decode
from test_gpu_decode import make_case

pytestmark = pytest.mark.gpu


def _both(dev, ranges, kernel=0):
    """(output through the caller's workspace, output through the static one)"""
    bt = dev.bt
    outs = []
    for static in (False, True):
        out = torch.full((bt.decoding_batches, bt.num_heads, bt.head_dim), float("nan"), dtype=torch.float16, device="cuda")
        plan, _ = dev.decode_only(num_token_ranges=ranges, output=out, static_workspace=static, kernel=kernel)
        torch.cuda.synchronize()
        outs.append(out)
    return outs[0], outs[1], plan


def test_static_workspace_entry_matches_the_workspace_entry(pkg, oracle):
    big = make_case(pkg, oracle, 601, num_heads=32, num_kv_heads=8, head_dim=128, cache_mode=1,
                    dec_kv_lens=[2100, 300, 17, 1290, 640, 2, 128, 999], outliers=True)
    small = make_case(pkg, oracle, 602, num_heads=32, num_kv_heads=8, head_dim=128, cache_mode=1,
                      dec_kv_lens=[500, 33, 260], outliers=True)
    mem_before = None
    for bt, dev, q, cache, scale in (big, small):  # the second call is the smaller one
        ref = oracle_decode(oracle, bt, q, cache, scale)
        for ranges in (0, 9):
            want, got, plan = _both(dev, ranges)
            assert plan.num_token_ranges > 1 and plan.workspace_size > 0
            assert not torch.isnan(got).any()
            assert torch.equal(want, got), "ranges %d: static workspace differs from the caller's workspace" % plan.num_token_ranges
            assert_attention_close(got.float().cpu().numpy(), ref, "static workspace, ranges %d" % plan.num_token_ranges)
        # no allocation through torch's allocator by the call itself (the output tensor above is the test's own)
        out = torch.empty((bt.decoding_batches, bt.num_heads, bt.head_dim), dtype=torch.float16, device="cuda")
        torch.cuda.synchronize()
        mem_before = torch.cuda.memory_allocated()
        dev.decode_only(num_token_ranges=9, output=out, static_workspace=True)
        torch.cuda.synchronize()
        assert torch.cuda.memory_allocated() == mem_before


def test_static_workspace_on_the_other_kernels(pkg, oracle):
    """The MFMA and the general kernel write their pieces the same way."""
    for seed, (hq, hkv, d) in ((611, (64, 8, 128)), (612, (8, 8, 64))):
        bt, dev, q, cache, scale = make_case(pkg, oracle, seed, num_heads=hq, num_kv_heads=hkv, head_dim=d, cache_mode=0,
                                             dec_kv_lens=[900, 300, 17], outliers=True)
        want, got, plan = _both(dev, 7)
        assert torch.equal(want, got)
        assert_attention_close(got.float().cpu().numpy(), oracle_decode(oracle, bt, q, cache, scale), str((hq, hkv, d)))


def test_static_workspace_rejects_what_does_not_fit(pkg, hip_lib):
    """Beyond the static array's size the call is refused on the host, before any launch."""
    L = pkg._lib
    p = L.DecodeParams()
    p.decoding_batches, p.num_heads, p.num_kv_heads, p.num_kv_repeats, p.head_dim = 4096, 64, 8, 8, 128
    p.num_token_ranges = 2048  # (2048 + 4096) * 64 * 130 * 4 bytes = 204 MB
    assert hip_lib.pmxhip_decode_attention_static(ctypes.byref(p), None) == L.PMXHIP_INVALID_VALUE
    assert b"static workspace" in hip_lib.pmxhip_last_error()
    need = (p.num_token_ranges + p.decoding_batches) * p.num_heads * (p.head_dim + 2) * 4
    assert need > L.STATIC_WORKSPACE_BYTES
