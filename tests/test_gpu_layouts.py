"""The cache layouts the reference's header documents, on the GPU through the C ABI.

The operator takes four free cache strides (multi_head_cache_attention.h:71-74) and its header names two orders of
the cache tensor, (S, L, 2, KVH, D) and (L, KVH, S, 2, D) (multi_head_cache_attention.h:145-146); the other GPU
tests use (L, 2, S, KVH, D).  Here every stage runs on the two documented orders against the oracle: the append
bit-exact, decode on every kernel family, prefill on the tile kernel and on the short-chunk route, and a mixed
forward(); and on a (L, KVH, S, 2, D) pool so large that the kv heads lie further apart than a 32-bit offset reaches.
Tolerance of the attention outputs: |got - ref| <= 2e-3 + 1e-2 * |ref|."""
import copy

import numpy as np
import pytest
import torch

from conftest import (assert_attention_close, host_cache, oracle_append_step, oracle_decode, oracle_fill_history,
                      oracle_prefill)

pytestmark = pytest.mark.gpu

LAYOUTS = ["sl2hd", "lhs2d"]
KERNEL_NAMES = {1: "decode_attention_kernel", 2: "decode_attention_quad_kernel",
                3: "decode_attention_mfma16_kernel", 4: "decode_attention_mfma_kernel"}


def _bits(a):
    return np.ascontiguousarray(a).view(np.uint16)


def test_layout_strides_are_the_documented_ones(pkg):
    lay = pkg.workloads.CacheLayout(3, 1000, 8, 128, "sl2hd")      # (S, L, 2, KVH, D)
    assert (lay.stride_s, lay.stride_l, lay.stride_kv, lay.stride_h) == (3 * 2 * 8 * 128, 2 * 8 * 128, 8 * 128, 128)
    lay = pkg.workloads.CacheLayout(3, 1000, 8, 128, "lhs2d")      # (L, KVH, S, 2, D)
    assert (lay.stride_l, lay.stride_h, lay.stride_s, lay.stride_kv) == (8 * 1000 * 2 * 128, 1000 * 2 * 128, 2 * 128, 128)
    lay = pkg.workloads.CacheLayout(3, 1000, 8, 128)               # (L, 2, S, KVH, D)
    assert (lay.stride_l, lay.stride_kv, lay.stride_s, lay.stride_h) == (2 * 1000 * 8 * 128, 1000 * 8 * 128, 8 * 128, 128)


@pytest.mark.parametrize("layout", LAYOUTS)
@pytest.mark.parametrize("cache_mode", [0, 1])
@pytest.mark.parametrize("heads", [(32, 8, 128), (8, 8, 64), (6, 3, 96), (8, 2, 256)])
def test_append_bit_exact(pkg, oracle, heads, cache_mode, layout):
    """Decode rows and prefill chunks appended into the middle layer of three: the whole cache and every scale,
    canaries of the other layers and of unowned rows included, equal the oracle's."""
    hq, hkv, d = heads
    bt, rng = pkg.workloads.custom_batch(500 + hq + d, num_heads=hq, num_kv_heads=hkv, head_dim=d, cache_mode=cache_mode,
                                         dec_kv_lens=[200, 4, 129, 1], prefill_q_lens=[10, 131, 1], prefill_prior=[125, 0, 300],
                                         num_layer=3, layer_idx=1, layout=layout)
    q, k, v = pkg.workloads.step_inputs(bt, rng)
    dev = pkg.harness.DeviceBatch(bt)
    dev.fill_canary()
    pkg.ops.key_value_cache(torch.from_numpy(k).cuda(), torch.from_numpy(v).cuda(), dev.seqstarts, dev.cachestarts,
                            dev.start_pos, dev.cache, dev.scale, batch=bt.batch, max_seqlen=bt.max_seqlen,
                            num_layer=bt.num_layer, layer_idx=bt.layer_idx, num_kv_heads=hkv, head_dim=d,
                            **dev.layout_kwargs())
    torch.cuda.synchronize()
    ref_c, ref_s = host_cache(bt, canary=(0x5A, 1.5))
    oracle_append_step(oracle, bt, k, v, ref_c, ref_s)
    assert np.array_equal(dev.cache.cpu().numpy(), ref_c)
    assert np.array_equal(_bits(dev.scale.cpu().numpy()), _bits(ref_s))


def make_case(pkg, oracle, seed, **kw):
    bt, rng = pkg.workloads.custom_batch(seed, **kw)
    cache, scale = host_cache(bt)
    oracle_fill_history(oracle, pkg, bt, rng, cache, scale)
    q, k, v = pkg.workloads.step_inputs(bt, rng)
    oracle_append_step(oracle, bt, k, v, cache, scale)
    dev = pkg.harness.DeviceBatch(bt)
    dev.cache.copy_(torch.from_numpy(cache))
    dev.scale.copy_(torch.from_numpy(scale))
    dev.set_step_inputs(q, k, v)
    return bt, dev, q, cache, scale


def run_decode(dev, ranges=0, **kw):
    dev.output.fill_(float("nan"))
    plan, ws = dev.decode_only(num_token_ranges=ranges, **kw)
    torch.cuda.synchronize()
    return dev.output[:dev.bt.decoding_batches].float().cpu().numpy(), plan


@pytest.mark.parametrize("layout", LAYOUTS)
@pytest.mark.parametrize("cache_mode", [0, 1])
@pytest.mark.parametrize("shape,kernels", [
    ((32, 8, 128), (0, 1, 2, 3, 4)),   # every kernel family on one shape
    ((64, 8, 128), (0, 2, 3)),         # two sets of waves of the quad kernel; the 16-column kernel by choice
    ((96, 4, 128), (0,)),              # 32 columns
    ((8, 8, 64), (0, 1)), ((128, 8, 64), (0,)), ((6, 2, 96), (0,)), ((16, 8, 256), (0, 1)), ((8, 1, 256), (0,)),
    ((5, 5, 128), (0, 1)), ((8, 1, 128), (0,)), ((71, 1, 64), (0,)),
])
def test_decode_matches_oracle(pkg, oracle, shape, kernels, cache_mode, layout):
    hq, hkv, d = shape
    bt, dev, q, cache, scale = make_case(pkg, oracle, 520 + hq + d, num_heads=hq, num_kv_heads=hkv, head_dim=d,
                                         cache_mode=cache_mode, dec_kv_lens=[1, 300, 17, 129, 640, 2, 128], outliers=True,
                                         num_layer=2, layer_idx=1, layout=layout)
    ref = oracle_decode(oracle, bt, q, cache, scale)
    for k in kernels:
        if k:
            assert dev.decode_only(kernel=k, name_only=True) == KERNEL_NAMES[k]
        for ranges in (1, 0, 5):
            got, plan = run_decode(dev, ranges, kernel=k)
            assert_attention_close(got, ref, "%s shape %s mode %d kernel %d ranges %d" % (layout, shape, cache_mode, k,
                                                                                          plan.num_token_ranges))


@pytest.mark.parametrize("layout", LAYOUTS)
def test_decode_with_mask(pkg, oracle, layout):
    hq, hkv, d = 32, 8, 128
    bt, dev, q, cache, scale = make_case(pkg, oracle, 531, num_heads=hq, num_kv_heads=hkv, head_dim=d, cache_mode=1,
                                         dec_kv_lens=[300, 17, 129, 640], outliers=True, layout=layout)
    rng = np.random.default_rng(5)
    cols = (int(bt.kvstarts[-1]) + 7) // 8 * 8
    mask = (rng.standard_normal((bt.decoding_batches, cols)) * 2.0).astype(np.float16)
    ref = oracle_decode(oracle, bt, q, cache, scale, attn_mask=mask, mask_stride_s=cols, mask_stride_h=0)
    md = torch.from_numpy(mask).cuda()
    for k in (0, 1, 3):
        got, _ = run_decode(dev, 0, kernel=k, attn_mask=md, mask_stride_s=cols, mask_stride_h=0)
        assert_attention_close(got, ref, "%s masked decode kernel %d" % (layout, k))


def run_prefill(pkg, dev, **extra):
    bt = dev.bt
    dev.output.fill_(float("nan"))
    pkg.ops.prefill_attention(dev.query, dev.output, dev.cache, dev.scale, dev.seqstarts, dev.kvstarts, dev.cachestarts,
                              attn_scale=bt.attn_scale, is_causal=bt.is_causal, batch=bt.batch,
                              decoding_batches=bt.decoding_batches, max_seqlen=bt.max_seqlen, max_kvlen=bt.max_kvlen,
                              layer_idx=bt.layer_idx, num_heads=bt.num_heads, num_kv_heads=bt.num_kv_heads,
                              head_dim=bt.head_dim, **dev.layout_kwargs(), **extra)
    torch.cuda.synchronize()
    return dev.output.float().cpu().numpy()


@pytest.mark.parametrize("layout", LAYOUTS)
@pytest.mark.parametrize("cache_mode", [0, 1])
@pytest.mark.parametrize("shape", [(8, 2, 128), (8, 8, 64), (8, 2, 256), (6, 6, 96)])
def test_prefill_tile_kernel(pkg, oracle, shape, cache_mode, layout):
    hq, hkv, d = shape
    bt, dev, q, cache, scale = make_case(pkg, oracle, 540 + hq + d, num_heads=hq, num_kv_heads=hkv, head_dim=d,
                                         cache_mode=cache_mode, dec_kv_lens=[33, 140],
                                         prefill_q_lens=[70, 7, 1, 129, 200], prefill_prior=[130, 0, 50, 127, 0],
                                         outliers=True, num_layer=2, layer_idx=1, layout=layout)
    ref = oracle_prefill(oracle, bt, q, cache, scale)
    got = run_prefill(pkg, dev)
    n_dec = bt.decoding_batches
    assert np.isnan(got[:n_dec]).all()
    assert_attention_close(got[n_dec:], ref[n_dec:], "%s prefill %s mode %d" % (layout, shape, cache_mode))


@pytest.mark.parametrize("layout", LAYOUTS)
@pytest.mark.parametrize("cache_mode", [0, 1])
@pytest.mark.parametrize("shape,q_lens", [((32, 8, 128), [4, 1, 8, 3, 2, 8, 5]), ((8, 8, 64), [16, 5, 32, 1, 31, 2, 9]),
                                          ((32, 8, 128), [4, 1, 2, 3, 4, 4, 1])])
def test_prefill_short_chunks_on_the_decode_kernel(pkg, oracle, shape, q_lens, cache_mode, layout):
    hq, hkv, d = shape
    bt, dev, q, cache, scale = make_case(pkg, oracle, 560 + hq + d, num_heads=hq, num_kv_heads=hkv, head_dim=d,
                                         cache_mode=cache_mode, dec_kv_lens=[33, 140], prefill_q_lens=q_lens,
                                         prefill_prior=[1500, 0, 900, 33, 2047, 126, 640], outliers=True, layout=layout)
    ref = oracle_prefill(oracle, bt, q, cache, scale)
    ws_bytes = pkg.ops.prefill_workspace_size(bt.batch, bt.decoding_batches, bt.max_seqlen, bt.max_kvlen, hq, hkv, d)
    assert ws_bytes > 0
    ws = torch.full((ws_bytes // 4,), float("nan"), dtype=torch.float32, device="cuda")
    got = run_prefill(pkg, dev, workspace=ws)
    assert_attention_close(got[bt.decoding_batches:], ref[bt.decoding_batches:], "%s chunks %s" % (layout, shape))
    assert not torch.isnan(ws).all()  # pieces were written: the decode step's kernel ran


@pytest.mark.parametrize("layout", LAYOUTS)
@pytest.mark.parametrize("heads,q_lens", [((32, 8, 128), [100, 17]), ((64, 8, 128), [100, 17]), ((8, 8, 64), [40, 200]),
                                          ((32, 8, 128), [4, 8])])
def test_mixed_forward(pkg, oracle, heads, q_lens, layout):
    """append + decode + prefill in one forward(), into the last of three layers: cache bit-exact, outputs in
    tolerance."""
    hq, hkv, d = heads
    bt, rng = pkg.workloads.custom_batch(580 + hq + d, num_heads=hq, num_kv_heads=hkv, head_dim=d, cache_mode=1,
                                         dec_kv_lens=[600, 33, 1500, 129, 1, 256], prefill_q_lens=q_lens,
                                         prefill_prior=[150, 0], outliers=True, num_layer=3, layer_idx=2, layout=layout)
    cache, scale = host_cache(bt, canary=(0x5A, 1.5))
    dev = pkg.harness.DeviceBatch(bt)
    dev.fill_canary()
    for b, pos, k_rows, v_rows in oracle_fill_history(oracle, pkg, bt, rng, cache, scale):
        dev.append_rows(b, pos, k_rows, v_rows)
    q, k, v = pkg.workloads.step_inputs(bt, rng)
    dev.set_step_inputs(q, k, v)
    dev.output.fill_(float("nan"))
    op = dev.make_operator()
    assert op.forward() == 0
    torch.cuda.synchronize()
    oracle_append_step(oracle, bt, k, v, cache, scale)
    assert np.array_equal(dev.cache.cpu().numpy(), cache)
    assert np.array_equal(_bits(dev.scale.cpu().numpy()), _bits(scale))
    ref = oracle_prefill(oracle, bt, q, cache, scale)
    ref[:bt.decoding_batches] = oracle_decode(oracle, bt, q, cache, scale)
    assert_attention_close(dev.output.float().cpu().numpy(), ref, "%s forward %s" % (layout, heads))


# ---- a (L, KVH, S, 2, D) pool whose kv heads lie gigabytes apart ------------------------------------------------

def _spread(pkg, bt, pool_tokens):
    """A copy of `bt` whose pages are spread evenly over a pool of `pool_tokens` tokens, and the map from its
    compact rows to the rows of the large pool."""
    page = pkg.workloads.PAGE
    small_pages = bt.layout.pool_tokens // page
    big_pages = pool_tokens // page
    page_map = np.round(np.linspace(0, big_pages - 1, small_pages)).astype(np.int64)
    assert len(np.unique(page_map)) == small_pages and page_map[-1] == big_pages - 1
    big = copy.copy(bt)
    big.cachestarts = page_map[bt.cachestarts // page] * page
    big.layout = pkg.workloads.CacheLayout(bt.num_layer, pool_tokens, bt.num_kv_heads, bt.head_dim, bt.layout.kind)
    small_rows = np.arange(small_pages * page)
    big_rows = page_map[small_rows // page] * page + small_rows % page
    return big, torch.from_numpy(small_rows).cuda(), torch.from_numpy(big_rows).cuda()


@pytest.mark.parametrize("pool_tokens,heads", [
    # eight kv heads of a workgroup span 2 GiB, two neighbours 256 MiB: the quad kernel, its wave's first head in the base
    ((1 << 20) + 128, (32, 8, 128)),
    # two neighbouring kv heads 2 GiB apart: kernels with a wave per kv head, the general kernel one kv head per workgroup
    ((1 << 23) + 128, (32, 8, 128)),
    ((1 << 24) + 128, (8, 4, 64)),
])
def test_kv_heads_further_apart_than_a_lane_offset(pkg, oracle, pool_tokens, heads):
    """No layout the reference documents is refused for its size: in (L, KVH, S, 2, D) cache_stride_h = S * 2 * D,
    so the kv heads of a large pool lie gigabytes apart.  The step's pages are spread over the whole pool (its last
    page is the pool's last); the compact pool of the same pages is the oracle's.  Append bit-exact on the touched
    rows and nothing written elsewhere; decode on every kernel that serves the shape, prefill on both routes."""
    hq, hkv, d = heads
    bt, rng = pkg.workloads.custom_batch(600 + hq + d, num_heads=hq, num_kv_heads=hkv, head_dim=d, cache_mode=1,
                                         dec_kv_lens=[600, 33, 1500, 129, 1, 256], prefill_q_lens=[100, 17, 4],
                                         prefill_prior=[150, 0, 700], outliers=True, layout="lhs2d")
    cache, scale = host_cache(bt)
    oracle_fill_history(oracle, pkg, bt, rng, cache, scale)
    q, k, v = pkg.workloads.step_inputs(bt, rng)
    big, small_rows, big_rows = _spread(pkg, bt, pool_tokens)
    span = hkv * big.layout.stride_h
    assert span >= 2 ** 31
    dev = pkg.harness.DeviceBatch(big)  # zero-filled
    lay = big.layout
    big_c, big_s = lay.canonical(dev.cache), lay.canonical(dev.scale)  # views [L, 2, S, H, D]
    small_lay = bt.layout
    big_c[:, :, big_rows] = small_lay.canonical(torch.from_numpy(cache).cuda())[:, :, small_rows]
    big_s[:, :, big_rows] = small_lay.canonical(torch.from_numpy(scale).cuda())[:, :, small_rows]
    dev.set_step_inputs(q, k, v)
    dev.output.fill_(float("nan"))
    op = dev.make_operator()
    assert op.forward() == 0
    torch.cuda.synchronize()

    oracle_append_step(oracle, bt, k, v, cache, scale)
    got_c = big_c[:, :, big_rows].cpu().numpy()
    got_s = big_s[:, :, big_rows].cpu().numpy()
    assert np.array_equal(got_c, small_lay.canonical(cache)[:, :, :len(small_rows)])
    assert np.array_equal(_bits(got_s), _bits(small_lay.canonical(scale)[:, :, :len(small_rows)]))
    ref = oracle_prefill(oracle, bt, q, cache, scale)
    n_dec = bt.decoding_batches
    ref_dec = oracle_decode(oracle, bt, q, cache, scale)
    ref[:n_dec] = ref_dec
    assert_attention_close(dev.output.float().cpu().numpy(), ref, "forward, heads %d bytes apart" % lay.stride_h)

    far = lay.stride_h >= 2 ** 31
    auto = dev.decode_only(name_only=True)
    if d == 128:
        assert auto == ("decode_attention_mfma16_kernel" if far else "decode_attention_quad_kernel")
    for kern in (0, 1, 2, 3, 4):
        if (kern == 3 and d != 128):
            continue
        if kern == 2 and far:  # the quad kernel's waves hold two kv heads: refused on request, with a message
            assert dev.decode_only(kernel=2, name_only=True) == ""
            assert "kv heads of a wave" in pkg._lib.last_error()
            continue
        for ranges in (0, 3):
            got, _ = run_decode(dev, ranges, kernel=kern)
            assert_attention_close(got, ref_dec, "decode kernel %d ranges %d" % (kern, ranges))
    # prefill: the tile kernel, and a step of short chunks on the decode step's kernel
    got = run_prefill(pkg, dev)
    assert_attention_close(got[n_dec:], ref[n_dec:], "tile kernel")
    bt2, rng2 = pkg.workloads.custom_batch(601, num_heads=hq, num_kv_heads=hkv, head_dim=d, cache_mode=1, dec_kv_lens=[33],
                                           prefill_q_lens=[4, 1, 8] if d == 128 else [16, 5, 9],
                                           prefill_prior=[1500, 0, 900], outliers=True, layout="lhs2d")
    cache2, scale2 = host_cache(bt2)
    oracle_fill_history(oracle, pkg, bt2, rng2, cache2, scale2)
    q2, k2, v2 = pkg.workloads.step_inputs(bt2, rng2)
    oracle_append_step(oracle, bt2, k2, v2, cache2, scale2)
    big2, small_rows2, big_rows2 = _spread(pkg, bt2, pool_tokens)
    # nothing outside the first step's rows was written: clear them and the pool is all zeros again
    big_c[:, :, big_rows] = 0
    big_s[:, :, big_rows] = 0
    assert not bool(dev.cache.any()) and not bool(dev.scale.any())
    dev2 = pkg.harness.DeviceBatch.__new__(pkg.harness.DeviceBatch)
    dev2.__dict__.update(dev.__dict__)
    dev2.bt = big2
    dev2.seqstarts = torch.from_numpy(big2.seqstarts).cuda()
    dev2.kvstarts = torch.from_numpy(big2.kvstarts).cuda()
    dev2.start_pos = torch.from_numpy(big2.start_pos).cuda()
    dev2.cachestarts = torch.from_numpy(np.ascontiguousarray(big2.cachestarts)).cuda()
    big_c[:, :, big_rows2] = bt2.layout.canonical(torch.from_numpy(cache2).cuda())[:, :, small_rows2]
    big_s[:, :, big_rows2] = bt2.layout.canonical(torch.from_numpy(scale2).cuda())[:, :, small_rows2]
    dev2.set_step_inputs(q2, k2, v2)
    ref2 = oracle_prefill(oracle, bt2, q2, cache2, scale2)
    ws_bytes = pkg.ops.prefill_workspace_size(bt2.batch, bt2.decoding_batches, bt2.max_seqlen, bt2.max_kvlen, hq, hkv, d)
    assert ws_bytes > 0
    ws = torch.full((ws_bytes // 4,), float("nan"), dtype=torch.float32, device="cuda")
    got2 = run_prefill(pkg, dev2, workspace=ws)
    assert_attention_close(got2[1:], ref2[1:], "short chunks on the decode kernel")
    assert not torch.isnan(ws).all()
