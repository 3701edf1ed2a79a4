"""Host-side checks that need no GPU: the C-ABI library loads and exports every
symbol the header declares, heuristic_prepare validates and derives what the
reference's does (utils.cu:68-131, 162-165, 210-214, 318-324), and the split plan
is sized consistently.  No kernel is launched."""
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "pmx_hip", "c_api.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"PMXHIP_API\s+[\w\s\*]+?\b(pmxhip_\w+)\s*\(", text)))


def test_library_exports_every_declared_symbol(pkg, hip_lib):
    names = declared_symbols()
    assert len(names) >= 17
    for n in names:
        assert hasattr(hip_lib, n), n
    assert sorted(pkg._lib.EXPORTED_SYMBOLS) == names
    assert b"gfx950" in hip_lib.pmxhip_version()


def base_args(**over):
    kw = dict(query_shape=(6, 32, 128), current_key_shape=(6, 8, 128), current_value_shape=(6, 8, 128),
              output_shape=(6, 32, 128), batch=6, decoding_batches=6, max_seqlen=1, max_kvlen=4096, layer_idx=0,
              num_layer=1, num_heads=32, num_kv_heads=8, head_dim=128, cache_mode=1, page_size=128,
              cache_stride_s=1024, cache_stride_l=2 * 1024 * 4096, cache_stride_h=128, cache_stride_kv=1024 * 4096,
              cachestarts_stride_b=32, compute_units_override=256)
    kw.update(over)
    return kw


def prepare(pkg, **over):
    op = pkg.ops.DynamicBatchingMultiHeadCacheAttention()
    return op, op.heuristic_prepare(**base_args(**over))


def test_prepare_derives_the_reference_values(pkg, hip_lib):
    op, rc = prepare(pkg)
    assert rc == pkg.ops.RC_SUCCESS
    c = op.cfg
    assert c.prefill_batches == 0
    assert (c.q_stride_s, c.k_stride_s, c.v_stride_s, c.o_stride_s) == (4096, 1024, 1024, 4096)
    assert c.num_kv_repeats == 4
    import numpy as np
    assert c.attn_scale == float(np.float32(1.0 / np.sqrt(np.float32(128))))
    assert c.decoding_algo == 3  # INFINITY_GQCA is what the reference would name for G = 4
    assert c.decoding_multi_block_counter_size == 0
    assert c.workspace_size == c.decoding_multi_block_partial_out_size + c.decoding_multi_block_partial_log_sum_exp_size
    # mask strides: 3-d and 2-d masks (utils.cu:117-126)
    op, rc = prepare(pkg, attn_mask=1 << 20, attn_mask_shape=(32, 6, 4104))
    assert rc == 0 and (op.cfg.mask_stride_h, op.cfg.mask_stride_s) == (6 * 4104, 4104)
    op, rc = prepare(pkg, attn_mask=1 << 20, attn_mask_shape=(6, 4104))
    assert rc == 0 and (op.cfg.mask_stride_h, op.cfg.mask_stride_s) == (0, 4104)
    op, rc = prepare(pkg, batch=9, decoding_batches=6)
    assert rc == 0 and op.cfg.prefill_batches == 3


@pytest.mark.parametrize("over,code", [
    (dict(query_shape=(6, 31, 128)), 2),          # leading dim on query heads
    (dict(output_shape=(6, 16, 128)), 2),
    (dict(current_key_shape=(6, 4, 128)), 2),
    (dict(current_value_shape=(6, 4, 128)), 2),
    (dict(page_size=64), 2),                      # paged mode needs 128-token pages
    (dict(num_heads=30, query_shape=(6, 30, 128), output_shape=(6, 30, 128)), 2),  # 30 % 8 != 0
    (dict(attn_mask=1 << 20, attn_mask_shape=(4104,)), 2),        # mask must be 2-d or 3-d
    (dict(attn_mask=1 << 20, attn_mask_shape=(6, 4100)), 2),      # last dim % 8
    (dict(specify_decoding_multi_block=3), 4),
    (dict(specify_decoding_multi_block=-1), 4),
    (dict(specify_decoding_tpb=128), 4),
    (dict(enable_sharemem_mhca=False, enable_infinity_mhca=False, enable_infinity_gqca=False), 1),  # no algorithm
    # prefill sequences at a head_dim the prefill stage does not have: refused before anything is enqueued
    (dict(batch=9, decoding_batches=6, max_seqlen=40, head_dim=80, query_shape=(90, 32, 80),
          current_key_shape=(90, 8, 80), current_value_shape=(90, 8, 80), output_shape=(90, 32, 80)), 2),
    (dict(batch=9, decoding_batches=6, max_seqlen=40, head_dim=32, query_shape=(90, 32, 32),
          current_key_shape=(90, 8, 32), current_value_shape=(90, 8, 32), output_shape=(90, 32, 32)), 2),
])
def test_prepare_error_branches(pkg, hip_lib, over, code):
    _, rc = prepare(pkg, **over)
    assert rc == code


def test_prepare_accepts_what_the_reference_accepts(pkg, hip_lib):
    for over in (dict(specify_decoding_tpb=256), dict(specify_decoding_tpb=512), dict(cache_mode=0, page_size=0),
                 dict(enable_infinity_gqca=False), dict(enable_sharemem_mhca=False),
                 dict(specify_decoding_multi_block=0), dict(specify_decoding_multi_block=2),
                 # decode-only batches take every head_dim of the decode kernels
                 dict(head_dim=256, query_shape=(6, 32, 256), current_key_shape=(6, 8, 256),
                      current_value_shape=(6, 8, 256), output_shape=(6, 32, 256)),
                 dict(head_dim=96, query_shape=(6, 32, 96), current_key_shape=(6, 8, 96),
                      current_value_shape=(6, 8, 96), output_shape=(6, 32, 96)),
                 # and batches with prefill sequences the four head dims of the reference's flash attention
                 dict(batch=9, decoding_batches=6, max_seqlen=40, head_dim=256, query_shape=(90, 32, 256),
                      current_key_shape=(90, 8, 256), current_value_shape=(90, 8, 256), output_shape=(90, 32, 256)),
                 dict(batch=9, decoding_batches=6, max_seqlen=40, head_dim=96, query_shape=(90, 32, 96),
                      current_key_shape=(90, 8, 96), current_value_shape=(90, 8, 96), output_shape=(90, 32, 96))):
        op, rc = prepare(pkg, **over)
        assert rc == 0, over
    op, _ = prepare(pkg, specify_decoding_multi_block=0)
    assert op.cfg.decoding_multi_block_size == 1 and op.cfg.workspace_size == 0
    op, _ = prepare(pkg, enable_infinity_gqca=False)
    assert op.cfg.decoding_algo == 1  # SHAREMEM_MHCA
    op, _ = prepare(pkg, enable_infinity_gqca=False, enable_sharemem_mhca=False)
    assert op.cfg.decoding_algo == 2  # INFINITY_MHCA


def test_forward_before_prepare_is_rejected(pkg, hip_lib):
    import ctypes
    h = hip_lib.pmxhip_mhca_create()
    try:
        assert hip_lib.pmxhip_mhca_set_workspace(h, None) == 4
        d = pkg._lib.MhcaDerived()
        assert hip_lib.pmxhip_mhca_get_derived(h, ctypes.byref(d)) == 4
    finally:
        hip_lib.pmxhip_mhca_destroy(h)


def test_decode_plan(pkg, hip_lib):
    plan = pkg.ops.decode_plan(128, 32, 8, 128, 8192, cus=256)
    assert plan.kv_heads_per_group == 8 and plan.q_heads_per_pass == 4 and plan.num_passes == 1
    assert plan.num_token_ranges == 256  # the quad kernel: a long stream is cut for one wave per SIMD
    pieces = plan.num_token_ranges + 128
    assert plan.partial_out_size == pieces * 32 * 128 * 4 and plan.partial_ml_size == pieces * 32 * 2 * 4
    plan = pkg.ops.decode_plan(64, 32, 32, 128, 4096, cus=256)  # MHA: 4 groups of 8 kv heads
    assert plan.kv_heads_per_group == 8 and plan.q_heads_per_pass == 1 and plan.num_token_ranges == 64
    plan = pkg.ops.decode_plan(32, 64, 8, 128, 32768, cus=256)  # G = 8: MFMA kernel, 4 kv heads per workgroup, 16 columns
    assert plan.q_heads_per_pass == 16 and plan.num_passes == 1 and plan.kv_heads_per_group == 4
    assert plan.num_token_ranges == 256
    plan = pkg.ops.decode_plan(64, 8, 1, 128, 8192, cus=256)  # one kv head: one wave per workgroup, eight workgroups per CU
    assert plan.q_heads_per_pass == 16 and plan.kv_heads_per_group == 1 and plan.num_token_ranges == 2048
    plan = pkg.ops.decode_plan(64, 16, 2, 128, 8192, cus=256)
    assert plan.q_heads_per_pass == 16 and plan.kv_heads_per_group == 2 and plan.num_token_ranges == 1024
    plan = pkg.ops.decode_plan(64, 16, 4, 128, 8192, cus=256)  # four kv heads: two waves per workgroup, four workgroups per CU
    assert plan.q_heads_per_pass == 4 and plan.kv_heads_per_group == 4 and plan.num_token_ranges == 1024
    plan = pkg.ops.decode_plan(4, 48, 3, 64, 512, cus=256)  # G = 16 at head_dim 64: 32 MFMA columns; 3 kv heads -> 1 per group
    assert plan.q_heads_per_pass == 32 and plan.num_passes == 1 and plan.kv_heads_per_group == 1
    plan = pkg.ops.decode_plan(4, 48, 3, 64, 512, cus=256, kernel=pkg._lib.DECODE_KERNEL_GENERAL)  # -> two passes of 8
    assert plan.q_heads_per_pass == 8 and plan.num_passes == 2 and plan.kv_heads_per_group == 1
    plan = pkg.ops.decode_plan(1, 8, 8, 64, 30, cus=256)    # tiny: one range, no workspace
    assert plan.num_token_ranges == 1 and plan.workspace_size == 0
    plan = pkg.ops.decode_plan(4, 8, 8, 64, 512, cus=256, ranges_hint=7)
    assert plan.num_token_ranges == 7
    with pytest.raises(pkg.ops.PmxError):
        pkg.ops.decode_plan(4, 8, 8, 80, 512, cus=256)  # head_dim 80
    with pytest.raises(pkg.ops.PmxError):
        pkg.ops.decode_plan(4, 9, 8, 64, 512, cus=256)


def test_decode_plan_names_its_kernel(pkg, hip_lib):
    """The plan reports the token-range kernel it was made for, and a requested kernel is honoured or refused."""
    L = pkg._lib
    auto = {(32, 8, 128): L.DECODE_KERNEL_QUAD, (32, 32, 128): L.DECODE_KERNEL_QUAD, (64, 8, 128): L.DECODE_KERNEL_MFMA16,
            (96, 4, 128): L.DECODE_KERNEL_MFMA32, (9, 3, 128): L.DECODE_KERNEL_QUAD, (6, 3, 128): L.DECODE_KERNEL_QUAD, (3, 1, 128): L.DECODE_KERNEL_MFMA16,
            (5, 5, 128): L.DECODE_KERNEL_QUAD, (2, 1, 128): L.DECODE_KERNEL_GENERAL, (3, 1, 64): L.DECODE_KERNEL_MFMA32,
            (8, 8, 64): L.DECODE_KERNEL_QUAD, (32, 8, 64): L.DECODE_KERNEL_QUAD, (40, 8, 64): L.DECODE_KERNEL_MFMA32,
            (9, 3, 64): L.DECODE_KERNEL_QUAD, (12, 4, 96): L.DECODE_KERNEL_GENERAL, (16, 16, 256): L.DECODE_KERNEL_QUAD,
            (40, 8, 256): L.DECODE_KERNEL_QUAD, (8, 1, 256): L.DECODE_KERNEL_QUAD, (72, 8, 256): L.DECODE_KERNEL_GENERAL, (66, 2, 128): L.DECODE_KERNEL_MFMA32, (48, 1, 128): L.DECODE_KERNEL_MFMA32,
            (71, 1, 64): L.DECODE_KERNEL_MFMA32, (2, 1, 64): L.DECODE_KERNEL_GENERAL}
    for (hq, hkv, d), want in auto.items():
        assert pkg.ops.decode_plan(16, hq, hkv, d, 4096, cus=256).kernel == want, (hq, hkv, d)
    # more than 32 query heads per kv head: passes of 32 columns (multi-query models)
    for (hq, hkv, d), passes in {(48, 1, 128): 2, (71, 1, 64): 3, (66, 2, 128): 2, (128, 4, 128): 1, (128, 8, 64): 1}.items():
        plan = pkg.ops.decode_plan(16, hq, hkv, d, 4096, cus=256)
        assert (plan.kernel, plan.q_heads_per_pass, plan.num_passes) == (L.DECODE_KERNEL_MFMA32, 32, passes), (hq, hkv, d)
    # requests: every kernel on the Llama-3-70B shape (8 query heads per kv head, kv heads in eights)
    for k, (kvhb, gt, ranges) in {L.DECODE_KERNEL_GENERAL: (8, 8, 512), L.DECODE_KERNEL_QUAD: (8, 8, 256),
                                  L.DECODE_KERNEL_MFMA16: (4, 16, 256), L.DECODE_KERNEL_MFMA32: (4, 32, 256)}.items():
        plan = pkg.ops.decode_plan(32, 64, 8, 128, 32768, cus=256, kernel=k)
        assert (plan.kernel, plan.kv_heads_per_group, plan.q_heads_per_pass, plan.num_token_ranges) == (k, kvhb, gt, ranges)
    for hq, hkv, d, k in [(40, 8, 64, L.DECODE_KERNEL_QUAD), (32, 8, 96, L.DECODE_KERNEL_QUAD), (32, 8, 64, L.DECODE_KERNEL_MFMA16),
                          (40, 2, 128, L.DECODE_KERNEL_MFMA16), (32, 8, 96, L.DECODE_KERNEL_MFMA32), (16, 4, 256, L.DECODE_KERNEL_MFMA32),
                          (10, 2, 128, L.DECODE_KERNEL_QUAD), (2, 1, 128, L.DECODE_KERNEL_QUAD), (32, 8, 128, 5), (32, 8, 128, -1)]:
        with pytest.raises(pkg.ops.PmxError):
            pkg.ops.decode_plan(16, hq, hkv, d, 4096, cus=256, kernel=k)


def test_c_entry_points_reject_bad_arguments_without_launching(pkg, hip_lib):
    """Argument checks run before any device work, so they can be exercised on the host."""
    import ctypes
    L = pkg._lib
    p = L.KvstoreParams()
    p.head_dim = 12
    p.num_kv_heads = 1
    p.batch = 1
    p.max_seqlen = 1
    assert hip_lib.pmxhip_kv_cache_quantize(ctypes.byref(p), None) == 2  # head_dim % 8 (kernel.cu:2040)
    p.head_dim = 64
    p.cache_mode = 2
    assert hip_lib.pmxhip_kv_cache_quantize(ctypes.byref(p), None) == 2  # invalid cache_mode (kernel.cu:2050)
    p.cache_mode = 1
    p.page_size = 64
    assert hip_lib.pmxhip_kv_cache_quantize(ctypes.byref(p), None) == 2
    p.page_size = 128
    p.cache_stride_s = 12
    assert hip_lib.pmxhip_kv_cache_quantize(ctypes.byref(p), None) == 2  # strides % 8
    p.cache_stride_s = 64
    assert hip_lib.pmxhip_kv_cache_quantize(ctypes.byref(p), None) == 4  # null pointers
    p.batch = 0
    assert hip_lib.pmxhip_kv_cache_quantize(ctypes.byref(p), None) == 0  # nothing to do
    assert hip_lib.pmxhip_kv_cache_quantize(None, None) == 4

    d = L.DecodeParams()
    assert hip_lib.pmxhip_decode_attention(ctypes.byref(d), None) == 0  # no decode sequences (kernel.cu:2084)
    d.decoding_batches = 2
    d.head_dim = 80
    assert hip_lib.pmxhip_decode_attention(ctypes.byref(d), None) == 2
    d.head_dim = 128
    d.num_heads, d.num_kv_heads, d.num_kv_repeats = 8, 3, 2
    assert hip_lib.pmxhip_decode_attention(ctypes.byref(d), None) == 2
    d.num_heads, d.num_kv_heads, d.num_kv_repeats = 8, 2, 4
    d.cache_mode = 3
    assert hip_lib.pmxhip_decode_attention(ctypes.byref(d), None) == 2
    d.cache_mode = 0
    assert hip_lib.pmxhip_decode_attention(ctypes.byref(d), None) == 4  # null pointers
    assert b"null" in hip_lib.pmxhip_last_error()

    f = L.PrefillParams()
    f.batch, f.decoding_batches = 2, 3
    assert hip_lib.pmxhip_prefill_attention(ctypes.byref(f), None) == 4
    f.batch, f.decoding_batches = 3, 3
    assert hip_lib.pmxhip_prefill_attention(ctypes.byref(f), None) == 0  # no prefill sequences (kernel.cu:2130)
    f.batch, f.max_seqlen, f.head_dim = 4, 8, 96
    assert hip_lib.pmxhip_prefill_attention(ctypes.byref(f), None) == 2


def test_bench_refuses_more_than_one_gpu():
    """bench.py measures one GPU; asking for more ends with a message that says so, before any device work."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode == 2
    assert "ONE GPU" in r.stderr and r.stdout.strip() == ""
