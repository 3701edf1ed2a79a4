"""TEST INFRASTRUCTURE ONLY -- Python face of the CPU oracle.

Loads ``libpmx_oracle.so`` (the C restatement in ``pmx_oracle.c``) through ctypes
and adds an independent numpy restatement of the quantiser so the two can be
checked against each other.  Only tests, the smoke check and the benchmark's
``cpu_baseline`` leg may import this module; the shipped library never does.

Reference lines restated: quantise/append = kernel.cu:86-157, decode semantics =
kernel.cu:299,347,404-415,509, prefill slicing = kernel.cu:2127-2179, causal
alignment = flash_attn2/src/mask.h:186, combine = kernel.cu:617-665 (all under
src/ppl/kernel/llm/cuda/ of the reference tree).
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libpmx_oracle.so")
_lib = None

_i64 = ctypes.c_int64
_i32 = ctypes.c_int32
_f32 = ctypes.c_float
_vp = ctypes.c_void_p


def build(force=False):
    """Compile the C oracle with gcc (seconds)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s", "libpmx_oracle.so"])
    return _LIB_PATH


def lib():
    global _lib
    if _lib is None:
        build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.pmx_oracle_half_to_float.restype = _f32
        _lib.pmx_oracle_half_to_float.argtypes = [ctypes.c_uint16]
        _lib.pmx_oracle_float_to_half.restype = ctypes.c_uint16
        _lib.pmx_oracle_float_to_half.argtypes = [_f32]
        _lib.pmx_oracle_quantize_group8.restype = None
        _lib.pmx_oracle_quantize_group8.argtypes = [_vp, _vp, _vp]
        _lib.pmx_oracle_kv_cache_quantize.restype = ctypes.c_int
        _lib.pmx_oracle_kv_cache_quantize.argtypes = [_vp] * 5 + [_i64] * 4 + [_i32] + [_i64] * 7 + [_vp] * 2
        _lib.pmx_oracle_decode_attention.restype = ctypes.c_int
        _lib.pmx_oracle_decode_attention.argtypes = (
            [_vp] * 6 + [_i64] * 4 + [_f32, _i64, _i32] + [_i64] * 9 + [_vp])
        _lib.pmx_oracle_prefill_attention.restype = ctypes.c_int
        _lib.pmx_oracle_prefill_attention.argtypes = (
            [_vp] * 6 + [_i64, _i64, _i32] + [_i64] * 3 + [_f32, _i64, _i32] + [_i64] * 7 + [_vp])
        _lib.pmx_oracle_prefill_attention_ex.restype = ctypes.c_int
        _lib.pmx_oracle_prefill_attention_ex.argtypes = (
            [_vp] * 5 + [_i64, _i64] + [_vp, _i64, _i64] + [_vp] + [_vp] * 3 + [_i64, _i64, _i32] + [_i64] * 3 +
            [_f32, _i64, _i32] + [_i64] * 7 + [_vp])
        _lib.pmx_oracle_decode_partial.restype = ctypes.c_int
        _lib.pmx_oracle_decode_partial.argtypes = (
            [_vp] * 4 + [_i64] * 7 + [_f32, _i64, _i32] + [_i64] * 6 + [_vp] * 3)
        _lib.pmx_oracle_splitkv_combine.restype = ctypes.c_int
        _lib.pmx_oracle_splitkv_combine.argtypes = [_vp] * 3 + [_i64, _i64, _vp]
        _lib.pmx_oracle_num_threads.restype = ctypes.c_int
        _lib.pmx_oracle_count_reciprocal_quotient_mismatches.restype = ctypes.c_int64
        _lib.pmx_oracle_count_reciprocal_quotient_mismatches.argtypes = [_vp]
        _lib.pmx_oracle_rotary_position_embedding.restype = ctypes.c_int
        _lib.pmx_oracle_rotary_position_embedding.argtypes = (
            [_vp] * 4 + [_f32, _i32] + [_i64] * 6 + [_i32, _f32] + [_i64] * 4 + [_vp] * 2)
        _lib.pmx_oracle_kv_cache_reorder.restype = ctypes.c_int
        _lib.pmx_oracle_kv_cache_reorder.argtypes = [_i32] + [_vp] * 6 + [_i64] * 8
        _lib.pmx_oracle_row_parallel_linear.restype = ctypes.c_int
        _lib.pmx_oracle_row_parallel_linear.argtypes = [_vp] * 3 + [_i64] * 6 + [_vp]
    return _lib


def _p(a):
    return None if a is None else a.ctypes.data_as(_vp)


def _c(a, dtype):
    a = np.ascontiguousarray(a, dtype=dtype)
    return a


# --------------------------------------------------------------------------
# independent numpy restatement of the quantiser (kernel.cu:128-148)
# --------------------------------------------------------------------------

def quantize_groups_numpy(x):
    """x: float16 array [..., 8].  Returns (int8 [..., 8], float16 scale [...]).

    Every numpy float16 operation is evaluated in a wider type and rounded once
    to binary16, i.e. it is the correctly rounded half operation the reference
    arithmetic denotes (absmax in half, scale via a float division, the half
    clamp to eps, the half quotient, round-half-even)."""
    x = np.asarray(x, dtype=np.float16)
    assert x.shape[-1] == 8
    eps = np.float16(np.float32(1e-5))
    amax = np.max(np.abs(x), axis=-1)
    s = (amax.astype(np.float32) / np.float32(127.0)).astype(np.float16)
    s = np.where(s > eps, s, eps).astype(np.float16)
    with np.errstate(over="ignore", invalid="ignore"):
        quo = (x.astype(np.float32) / s[..., None].astype(np.float32)).astype(np.float16)
    q = np.rint(quo.astype(np.float32)).astype(np.int32).astype(np.int8)
    return q, s


def quantize_groups_c(x):
    """Same contract as quantize_groups_numpy, through the C oracle."""
    x = _c(x, np.float16)
    flat = x.reshape(-1, 8)
    q = np.empty(flat.shape, dtype=np.int8)
    s = np.empty(flat.shape[0], dtype=np.float16)
    fn = lib().pmx_oracle_quantize_group8
    xb = flat.view(np.uint16)
    for i in range(flat.shape[0]):
        fn(xb[i].ctypes.data, q[i].ctypes.data, s[i:i + 1].ctypes.data)
    return q.reshape(x.shape), s.reshape(x.shape[:-1])


# --------------------------------------------------------------------------
# stage wrappers (arguments follow the reference's kernel parameter structs)
# --------------------------------------------------------------------------

def kv_cache_quantize(current_key, current_value, seqstarts, cachestarts, start_pos,
                      layer_idx, num_kv_heads, head_dim, page_size,
                      cache_stride_s, cache_stride_l, cache_stride_h, cache_stride_kv,
                      cachestarts_stride_b, cache, scale,
                      key_stride_s=None, value_stride_s=None):
    """In-place append into ``cache`` (int8) / ``scale`` (float16)."""
    assert current_key.dtype == np.float16 and current_value.dtype == np.float16
    assert cache.dtype == np.int8 and scale.dtype == np.float16
    assert cache.flags.c_contiguous and scale.flags.c_contiguous
    current_key = _c(current_key, np.float16)
    current_value = _c(current_value, np.float16)
    seqstarts = _c(seqstarts, np.int64)
    cachestarts = _c(cachestarts, np.int64)
    start_pos = _c(start_pos, np.int64)
    batch = seqstarts.shape[0] - 1
    ks = num_kv_heads * head_dim if key_stride_s is None else key_stride_s
    vs = num_kv_heads * head_dim if value_stride_s is None else value_stride_s
    rc = lib().pmx_oracle_kv_cache_quantize(
        _p(current_key), _p(current_value), _p(seqstarts), _p(cachestarts), _p(start_pos),
        batch, layer_idx, num_kv_heads, head_dim, page_size, ks, vs,
        cache_stride_s, cache_stride_l, cache_stride_h, cache_stride_kv, cachestarts_stride_b,
        _p(cache), _p(scale))
    if rc != 0:
        raise ValueError("oracle quantize rejected the arguments (rc=%d)" % rc)


def decode_attention(query, cache, scale, cachestarts, kvstarts, decoding_batches,
                     num_heads, num_kv_heads, head_dim, attn_scale, layer_idx, page_size,
                     cache_stride_s, cache_stride_l, cache_stride_h, cache_stride_kv,
                     cachestarts_stride_b, attn_mask=None, mask_stride_s=0, mask_stride_h=0):
    """Returns float32 [decoding_batches, num_heads, head_dim]."""
    query = _c(query, np.float16)
    cachestarts = _c(cachestarts, np.int64)
    kvstarts = _c(kvstarts, np.int64)
    if attn_mask is not None:
        attn_mask = _c(attn_mask, np.float16)
    out = np.zeros((decoding_batches, num_heads, head_dim), dtype=np.float32)
    stride = num_heads * head_dim
    rc = lib().pmx_oracle_decode_attention(
        _p(query), _p(attn_mask), _p(cache), _p(scale), _p(cachestarts), _p(kvstarts),
        decoding_batches, num_heads, num_kv_heads, head_dim,
        attn_scale, layer_idx, page_size,
        stride, stride, mask_stride_s, mask_stride_h,
        cache_stride_s, cache_stride_l, cache_stride_h, cache_stride_kv, cachestarts_stride_b,
        _p(out))
    if rc != 0:
        raise ValueError("oracle decode rejected the arguments (rc=%d)" % rc)
    return out


def prefill_attention(query, cache, scale, seqstarts, kvstarts, cachestarts, batch,
                      decoding_batches, is_causal, num_heads, num_kv_heads, head_dim,
                      attn_scale, layer_idx, page_size,
                      cache_stride_s, cache_stride_l, cache_stride_h, cache_stride_kv,
                      cachestarts_stride_b):
    """Returns float32 [total_query_rows, num_heads, head_dim]; decode rows stay 0."""
    query = _c(query, np.float16)
    seqstarts = _c(seqstarts, np.int64)
    kvstarts = _c(kvstarts, np.int64)
    cachestarts = _c(cachestarts, np.int64)
    out = np.zeros((query.shape[0], num_heads, head_dim), dtype=np.float32)
    stride = num_heads * head_dim
    rc = lib().pmx_oracle_prefill_attention(
        _p(query), _p(cache), _p(scale), _p(seqstarts), _p(kvstarts), _p(cachestarts),
        batch, decoding_batches, 1 if is_causal else 0, num_heads, num_kv_heads, head_dim,
        attn_scale, layer_idx, page_size, stride, stride,
        cache_stride_s, cache_stride_l, cache_stride_h, cache_stride_kv, cachestarts_stride_b,
        _p(out))
    if rc != 0:
        raise ValueError("oracle prefill rejected the arguments (rc=%d)" % rc)
    return out


def prefill_attention_ex(query, cache, scale, seqstarts, kvstarts, cachestarts, batch,
                         decoding_batches, is_causal, num_heads, num_kv_heads, head_dim,
                         attn_scale, layer_idx, page_size,
                         cache_stride_s, cache_stride_l, cache_stride_h, cache_stride_kv,
                         cachestarts_stride_b, current_key=None, current_value=None,
                         attn_mask=None, mask_stride_s=0, mask_stride_h=0, alibi_slopes=None):
    """Prefill with the optional inputs: fp16 current_key/current_value [rows, KVH, D] instead of
    the cache, additive fp16 attn_mask, float32 alibi_slopes [Hq].  Returns float32
    [total_query_rows, num_heads, head_dim]; decode rows stay 0."""
    query = _c(query, np.float16)
    seqstarts = _c(seqstarts, np.int64)
    kvstarts = _c(kvstarts, np.int64)
    cachestarts = _c(cachestarts, np.int64)
    ck = None if current_key is None else _c(current_key, np.float16)
    cv = None if current_value is None else _c(current_value, np.float16)
    am = None if attn_mask is None else _c(attn_mask, np.float16)
    al = None if alibi_slopes is None else _c(alibi_slopes, np.float32)
    out = np.zeros((query.shape[0], num_heads, head_dim), dtype=np.float32)
    stride = num_heads * head_dim
    kstride = num_kv_heads * head_dim
    rc = lib().pmx_oracle_prefill_attention_ex(
        _p(query), _p(cache), _p(scale), _p(ck), _p(cv), kstride, kstride,
        _p(am), mask_stride_s, mask_stride_h, _p(al),
        _p(seqstarts), _p(kvstarts), _p(cachestarts),
        batch, decoding_batches, 1 if is_causal else 0, num_heads, num_kv_heads, head_dim,
        attn_scale, layer_idx, page_size, stride, stride,
        cache_stride_s, cache_stride_l, cache_stride_h, cache_stride_kv, cachestarts_stride_b,
        _p(out))
    if rc != 0:
        raise ValueError("oracle prefill rejected the arguments (rc=%d)" % rc)
    return out


def decode_partial(query, cache, scale, cachestarts, b, h, kv_begin, kv_end,
                   num_heads, num_kv_heads, head_dim, attn_scale, layer_idx, page_size,
                   cache_stride_s, cache_stride_l, cache_stride_h, cache_stride_kv,
                   cachestarts_stride_b):
    """Attention of (sequence b, head h) over kv positions [kv_begin, kv_end).
    Returns (normalised partial out float32[D], running max, exp-sum)."""
    query = _c(query, np.float16)
    cachestarts = _c(cachestarts, np.int64)
    out = np.zeros(head_dim, dtype=np.float32)
    mx = np.zeros(1, dtype=np.float32)
    sm = np.zeros(1, dtype=np.float32)
    lib().pmx_oracle_decode_partial(
        _p(query), _p(cache), _p(scale), _p(cachestarts), b, h, kv_begin, kv_end,
        num_heads, num_kv_heads, head_dim, attn_scale, layer_idx, page_size,
        num_heads * head_dim,
        cache_stride_s, cache_stride_l, cache_stride_h, cache_stride_kv, cachestarts_stride_b,
        _p(out), _p(mx), _p(sm))
    return out, float(mx[0]), float(sm[0])


def splitkv_combine(partial_out, partial_max, partial_sum):
    partial_out = _c(partial_out, np.float32)
    partial_max = _c(partial_max, np.float32)
    partial_sum = _c(partial_sum, np.float32)
    n, d = partial_out.shape
    out = np.zeros(d, dtype=np.float32)
    lib().pmx_oracle_splitkv_combine(_p(partial_out), _p(partial_max), _p(partial_sum), n, d, _p(out))
    return out


def count_reciprocal_quotient_mismatches():
    """(pairs whose int8 results differ, pairs whose half quotients differ in bits) over every
    finite half numerator and every half scale >= eps."""
    half_differs = ctypes.c_int64(0)
    bad = lib().pmx_oracle_count_reciprocal_quotient_mismatches(ctypes.byref(half_differs))
    return int(bad), int(half_differs.value)


def num_threads():
    return int(lib().pmx_oracle_num_threads())


def kv_cache_reorder(invert, kv_cache, kv_scale, outer_mem, page_ids, src_stride, dst_stride, layers, kv_heads, tokens,
                     head_dim, group_size, tp_rank, tp_size):
    """In place on the uint8 numpy arrays: gathers pages into outer_mem (invert=False) or scatters them back
    into kv_cache / kv_scale (invert=True).  Strides: 12 ints, {p, l, kv, h, t, d} for cache then scale."""
    assert kv_cache.dtype == np.uint8 and kv_scale.dtype == np.uint8 and outer_mem.dtype == np.uint8
    page_ids = _c(page_ids, np.int64)
    ss = _c(src_stride, np.int32)
    ds = _c(dst_stride, np.int32)
    lib().pmx_oracle_kv_cache_reorder(1 if invert else 0, _p(kv_cache), _p(kv_scale), _p(outer_mem), _p(page_ids),
                                      _p(ss), _p(ds), len(page_ids), layers, kv_heads, tokens, head_dim, group_size,
                                      tp_rank, tp_size)


def rotary_position_embedding(query, key, start_pos, seqstarts, theta, rotary_dim, bypass_key=False,
                              max_position_embeddings=2048, scaling_type=0, scaling_factor=1.0):
    """query [S, Hq, D], key [S, KVH, D] float16 -> (rotated_query, rotated_key) float16."""
    query = _c(query, np.float16)
    key = _c(key, np.float16)
    start_pos = _c(start_pos, np.int64)
    seqstarts = _c(seqstarts, np.int64)
    rq = np.zeros_like(query)
    rk = np.zeros_like(key)
    hq, d = query.shape[1], query.shape[2]
    hk = key.shape[1]
    rc = lib().pmx_oracle_rotary_position_embedding(
        _p(query), _p(key), _p(start_pos), _p(seqstarts), theta, 1 if bypass_key else 0, rotary_dim,
        len(start_pos), hq, hk, d, max_position_embeddings, scaling_type, scaling_factor,
        hq * d, hk * d, hq * d, hk * d, _p(rq), _p(rk))
    if rc != 0:
        raise ValueError("oracle rope rejected the arguments (rc=%d)" % rc)
    return rq, rk


def row_parallel_linear(input, weight, bias=None):
    """input [M, K], weight [N, K], bias [N] or None, all float16 -> output [M, N] float16 (float32 accumulate)."""
    input = _c(input, np.float16)
    weight = _c(weight, np.float16)
    m, k = input.shape
    n = weight.shape[0]
    assert weight.shape[1] == k
    b = _c(bias, np.float16) if bias is not None else None
    out = np.zeros((m, n), dtype=np.float16)
    rc = lib().pmx_oracle_row_parallel_linear(_p(input), _p(weight), _p(b) if b is not None else None, m, n, k, k, k, n, _p(out))
    if rc != 0:
        raise ValueError("oracle row_parallel_linear rejected the arguments (rc=%d)" % rc)
    return out
