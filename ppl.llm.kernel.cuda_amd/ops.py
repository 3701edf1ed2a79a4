"""Host-side mirror of the pmx operator interface over the C ABI.

Tensors are torch tensors that live in GPU memory; torch is used for nothing but
allocation and the current stream.  Every function goes through
libpmx_hip.so -- there is no PyTorch or CPU implementation behind these names.

Names follow the reference operator
(include/ppl/kernel/llm/cuda/pmx/multi_head_cache_attention.h:25-159):
``DynamicBatchingMultiHeadCacheAttention.heuristic_prepare / forward_kvstore /
forward_decode / forward_prefill / forward``; ``key_value_cache`` is the append
step as a free function.
"""
import ctypes

import torch

from . import _lib
from ._lib import (DATATYPE_FLOAT16, DecodeParams, DecodePlan, KvstoreParams, MhcaDerived,
                   MhcaPrepareArgs, PrefillParams, TensorShape)

RC_SUCCESS = _lib.PMXHIP_SUCCESS
RC_OTHER_ERROR = _lib.PMXHIP_OTHER_ERROR
RC_UNSUPPORTED = _lib.PMXHIP_UNSUPPORTED
RC_INVALID_VALUE = _lib.PMXHIP_INVALID_VALUE


class PmxError(RuntimeError):
    def __init__(self, code, where):
        self.code = code
        super().__init__("%s failed with status %d: %s" % (where, code, _lib.last_error()))


def _ptr(t):
    if t is None:
        return None
    if isinstance(t, int):
        return t
    if not t.is_cuda:
        raise ValueError("device tensor expected (got a CPU tensor)")
    return t.data_ptr()


def _stream(stream=None):
    if stream is None:
        stream = torch.cuda.current_stream()
    return ctypes.c_void_p(stream.cuda_stream)


def compute_units(device=None):
    return torch.cuda.get_device_properties(device if device is not None else torch.cuda.current_device()).multi_processor_count


def key_value_cache(current_key, current_value, seqstarts, cachestarts, start_pos, cache, scale, *,
                    batch, max_seqlen, num_layer, layer_idx, num_kv_heads, head_dim, cache_mode, page_size,
                    cache_stride_s, cache_stride_l, cache_stride_h, cache_stride_kv, cachestarts_stride_b,
                    stream=None, check=True):
    """Quantise/append `current_key`/`current_value` (fp16 [S, KVH, D]) into the int8 cache."""
    p = KvstoreParams()
    p.current_key = _ptr(current_key)
    p.current_value = _ptr(current_value)
    p.seqstarts = _ptr(seqstarts)
    p.cachestarts = _ptr(cachestarts)
    p.start_pos = _ptr(start_pos)
    p.num_layer = num_layer
    p.layer_idx = layer_idx
    p.num_kv_heads = num_kv_heads
    p.head_dim = head_dim
    p.page_size = page_size
    p.current_key_stride_s = num_kv_heads * head_dim
    p.current_value_stride_s = num_kv_heads * head_dim
    p.cache_stride_s = cache_stride_s
    p.cache_stride_l = cache_stride_l
    p.cache_stride_h = cache_stride_h
    p.cache_stride_kv = cache_stride_kv
    p.cachestarts_stride_b = cachestarts_stride_b
    p.cache = _ptr(cache)
    p.scale = _ptr(scale)
    p.batch = batch
    p.max_seqlen = max_seqlen
    p.cache_mode = cache_mode
    rc = _lib.lib().pmxhip_kv_cache_quantize(ctypes.byref(p), _stream(stream))
    if check and rc != RC_SUCCESS:
        raise PmxError(rc, "key_value_cache")
    return rc


def init():
    """The library's one-time set-up on the current device (needed only before a first step under stream capture)."""
    rc = _lib.lib().pmxhip_init()
    if rc != RC_SUCCESS:
        raise PmxError(rc, "init")
    return rc


def decode_plan(decoding_batches, num_heads, num_kv_heads, head_dim, max_kvlen, cus=None, ranges_hint=0, kernel=0):
    """The split plan of a decode step; `kernel` requests a token-range kernel (0 = chosen by shape)."""
    plan = DecodePlan()
    rc = _lib.lib().pmxhip_decode_plan_make_kernel(decoding_batches, num_heads, num_kv_heads, head_dim, max_kvlen,
                                                   compute_units() if cus is None else cus, ranges_hint, kernel,
                                                   ctypes.byref(plan))
    if rc != RC_SUCCESS:
        raise PmxError(rc, "decode_plan")
    return plan


def decode_attention(query, output, cache, scale, cachestarts, kvstarts, *, attn_scale, layer_idx,
                     decoding_batches, num_heads, num_kv_heads, head_dim, cache_mode, page_size,
                     cache_stride_s, cache_stride_l, cache_stride_h, cache_stride_kv, cachestarts_stride_b,
                     num_token_ranges, workspace=None, attn_mask=None, mask_stride_s=0, mask_stride_h=0,
                     stage=0, stream=None, check=True, kernel=0, static_workspace=False, output_stride_s=None,
                     name_only=False):
    """Decode attention of sequences [0, decoding_batches); output fp16 [B_dec, Hq, D].
    `kernel` requests a token-range kernel; `static_workspace` goes through the entry point that allocates
    nothing (the library's own workspace); `name_only` launches nothing and returns the kernel's name."""
    p = DecodeParams()
    p.query = _ptr(query)
    p.attn_mask = _ptr(attn_mask)
    p.output = _ptr(output)
    p.cache = _ptr(cache)
    p.scale = _ptr(scale)
    p.cachestarts = _ptr(cachestarts)
    p.kvstarts = _ptr(kvstarts)
    p.attn_scale = attn_scale
    p.layer_idx = layer_idx
    p.num_kv_repeats = num_heads // num_kv_heads if num_kv_heads else 0
    p.page_size = page_size
    p.query_stride_s = num_heads * head_dim
    p.output_stride_s = num_heads * head_dim if output_stride_s is None else output_stride_s
    p.mask_stride_s = mask_stride_s
    p.mask_stride_h = mask_stride_h
    p.cache_stride_s = cache_stride_s
    p.cache_stride_l = cache_stride_l
    p.cache_stride_h = cache_stride_h
    p.cache_stride_kv = cache_stride_kv
    p.cachestarts_stride_b = cachestarts_stride_b
    p.decoding_batches = decoding_batches
    p.num_heads = num_heads
    p.num_kv_heads = num_kv_heads
    p.head_dim = head_dim
    p.cache_mode = cache_mode
    p.num_token_ranges = num_token_ranges
    p.workspace = _ptr(workspace)
    p.workspace_size = 0 if workspace is None else workspace.numel() * workspace.element_size()
    p.kernel_request = kernel
    if name_only:
        return _lib.lib().pmxhip_decode_kernel_name(ctypes.byref(p)).decode()
    if static_workspace:
        if stage != 0:
            raise ValueError("the static-workspace entry point runs both stages")
        rc = _lib.lib().pmxhip_decode_attention_static(ctypes.byref(p), _stream(stream))
    else:
        rc = _lib.lib().pmxhip_decode_attention_stage(ctypes.byref(p), stage, _stream(stream))
    if check and rc != RC_SUCCESS:
        raise PmxError(rc, "decode_attention")
    return rc


def splitkv_combine(partial_out, partial_ml, piece_begin, piece_end, output, *, head_dim, stream=None):
    rows = piece_begin.numel()
    rc = _lib.lib().pmxhip_splitkv_combine(_ptr(partial_out), _ptr(partial_ml), _ptr(piece_begin), _ptr(piece_end),
                                           rows, head_dim, _ptr(output), _stream(stream))
    if rc != RC_SUCCESS:
        raise PmxError(rc, "splitkv_combine")
    return rc


def prefill_attention(query, output, cache, scale, seqstarts, kvstarts, cachestarts, *, attn_scale, is_causal,
                      batch, decoding_batches, max_seqlen, max_kvlen, layer_idx, num_heads, num_kv_heads,
                      head_dim, cache_mode, page_size, cache_stride_s, cache_stride_l, cache_stride_h,
                      cache_stride_kv, cachestarts_stride_b, attn_mask=None, mask_stride_s=0, mask_stride_h=0,
                      alibi_slopes=None, current_key=None, current_value=None, prefill_query_rows=None, workspace=None,
                      stream=None, check=True):
    """Multi-query-token attention of the prefill sequences.  Optional: additive half `attn_mask` with its
    strides, float32 `alibi_slopes` [Hq], `current_key`/`current_value` [rows, KVH, D] to attend over
    the step's own fp16 rows instead of the cache, and a `workspace` of prefill_workspace_size() bytes with which a
    batch of short chunks runs on the decode step's kernel."""
    p = PrefillParams()
    p.query = _ptr(query)
    p.output = _ptr(output)
    p.cache = _ptr(cache)
    p.scale = _ptr(scale)
    p.seqstarts = _ptr(seqstarts)
    p.kvstarts = _ptr(kvstarts)
    p.cachestarts = _ptr(cachestarts)
    p.attn_scale = attn_scale
    p.is_causal = 1 if is_causal else 0
    p.batch = batch
    p.decoding_batches = decoding_batches
    p.max_seqlen = max_seqlen
    p.max_kvlen = max_kvlen
    p.layer_idx = layer_idx
    p.num_heads = num_heads
    p.num_kv_heads = num_kv_heads
    p.head_dim = head_dim
    p.cache_mode = cache_mode
    p.page_size = page_size
    p.query_stride_s = num_heads * head_dim
    p.output_stride_s = num_heads * head_dim
    p.cache_stride_s = cache_stride_s
    p.cache_stride_l = cache_stride_l
    p.cache_stride_h = cache_stride_h
    p.cache_stride_kv = cache_stride_kv
    p.cachestarts_stride_b = cachestarts_stride_b
    p.attn_mask = _ptr(attn_mask) if attn_mask is not None else None
    p.mask_stride_s = mask_stride_s
    p.mask_stride_h = mask_stride_h
    p.alibi_slopes = _ptr(alibi_slopes) if alibi_slopes is not None else None
    if current_key is not None:
        p.current_key = _ptr(current_key)
        p.current_value = _ptr(current_value)
        p.key_stride_s = num_kv_heads * head_dim
        p.value_stride_s = num_kv_heads * head_dim
    # the rows of the prefill sequences follow from the query tensor (decode sequences have one row each)
    p.prefill_query_rows = (int(query.shape[0]) - decoding_batches) if prefill_query_rows is None else prefill_query_rows
    if workspace is not None:
        p.workspace = _ptr(workspace)
        p.workspace_size = int(workspace.numel() * workspace.element_size())
    rc = _lib.lib().pmxhip_prefill_attention(ctypes.byref(p), _stream(stream))
    if check and rc != RC_SUCCESS:
        raise PmxError(rc, "prefill_attention")
    return rc


def prefill_workspace_size(batch, decoding_batches, max_seqlen, max_kvlen, num_heads, num_kv_heads, head_dim, cus=0):
    """Bytes of the workspace with which a batch of short chunks runs on the decode step's kernel; 0 for every
    other batch (cus = 0: the compute units of the current device)."""
    return int(_lib.lib().pmxhip_prefill_workspace_size(batch, decoding_batches, max_seqlen, max_kvlen, num_heads,
                                                        num_kv_heads, head_dim, cus))


def _rope_params(query, key, start_pos, seqstarts, rotated_query, rotated_key, *, theta, rotary_dim, batch, max_seqlen,
                 bypass_key=False, max_position_embeddings=2048, scaling_type=0, scaling_factor=1.0):
    p = _lib.RopeParams()
    hq, d = int(query.shape[1]), int(query.shape[2])
    hk = int(key.shape[1])
    p.query, p.key = _ptr(query), _ptr(key)
    p.start_pos, p.seqstarts = _ptr(start_pos), _ptr(seqstarts)
    p.theta, p.bypass_key, p.rotary_dim, p.batch = theta, 1 if bypass_key else 0, rotary_dim, batch
    p.num_heads, p.num_key_heads, p.head_dim, p.max_seqlen = hq, hk, d, max_seqlen
    p.max_position_embeddings, p.scaling_type, p.scaling_factor = max_position_embeddings, scaling_type, scaling_factor
    p.query_stride_s = p.rotated_query_stride_s = hq * d
    p.key_stride_s = p.rotated_key_stride_s = hk * d
    p.rotated_query = _ptr(rotated_query)
    p.rotated_key = _ptr(rotated_key) if rotated_key is not None else None
    return p


def rotary_position_embedding(query, key, start_pos, seqstarts, rotated_query, rotated_key, *, stream=None, check=True, **kw):
    """Rotates the channel pairs of `query` [S, Hq, D] and `key` [S, KVH, D] (fp16) by their positions."""
    p = _rope_params(query, key, start_pos, seqstarts, rotated_query, rotated_key, **kw)
    rc = _lib.lib().pmxhip_rotary_position_embedding(ctypes.byref(p), _stream(stream))
    if check and rc != RC_SUCCESS:
        raise PmxError(rc, "rotary_position_embedding")
    return rc


def rope_key_value_cache(query, key, value, start_pos, seqstarts, cachestarts, rotated_query, rotated_key, cache, scale, *,
                         num_layer, layer_idx, cache_mode, page_size, cache_stride_s, cache_stride_l, cache_stride_h,
                         cache_stride_kv, cachestarts_stride_b, stream=None, check=True, **kw):
    """The rotation and, in the same kernel, the quantise/append of the rotated key and of `value`;
    `rotated_key` may be None."""
    p = _rope_params(query, key, start_pos, seqstarts, rotated_query, rotated_key, **kw)
    st = KvstoreParams()
    st.current_key, st.current_value = _ptr(key), _ptr(value)
    st.seqstarts, st.cachestarts, st.start_pos = _ptr(seqstarts), _ptr(cachestarts), _ptr(start_pos)
    st.num_layer, st.layer_idx = num_layer, layer_idx
    st.num_kv_heads, st.head_dim, st.page_size = p.num_key_heads, p.head_dim, page_size
    st.current_key_stride_s = st.current_value_stride_s = p.key_stride_s
    st.cache_stride_s, st.cache_stride_l, st.cache_stride_h = cache_stride_s, cache_stride_l, cache_stride_h
    st.cache_stride_kv, st.cachestarts_stride_b = cache_stride_kv, cachestarts_stride_b
    st.cache, st.scale = _ptr(cache), _ptr(scale)
    st.batch, st.max_seqlen, st.cache_mode = p.batch, p.max_seqlen, cache_mode
    rc = _lib.lib().pmxhip_rope_kv_cache_quantize(ctypes.byref(p), ctypes.byref(st), _stream(stream))
    if check and rc != RC_SUCCESS:
        raise PmxError(rc, "rope_kv_cache_quantize")
    return rc


def kv_cache_reorder(kv_cache, kv_scale, page_ids, src_stride, dst_stride, *, layers, kv_heads, tokens, head_dim,
                     group_size, tp_rank, tp_size, outer_mem, stream=None, check=True):
    """Gathers the pages `page_ids` of the int8 cache and of its scales into `outer_mem`.
    Strides: 12 byte strides, {page, layer, plane, head, token, byte} of the cache then of the scales."""
    s, d = _lib.ReorderStride.of(src_stride), _lib.ReorderStride.of(dst_stride)
    rc = _lib.lib().pmxhip_kv_cache_reorder(_stream(stream), _ptr(kv_cache), _ptr(kv_scale), _ptr(page_ids),
                                            ctypes.byref(s), ctypes.byref(d), int(page_ids.numel()), layers, kv_heads,
                                            tokens, head_dim, group_size, tp_rank, tp_size, _ptr(outer_mem))
    if check and rc != RC_SUCCESS:
        raise PmxError(rc, "kv_cache_reorder")
    return rc


def kv_cache_invert_reorder(outer_mem, page_ids, src_stride, dst_stride, *, layers, kv_heads, tokens, head_dim,
                            group_size, tp_rank, tp_size, kv_cache, kv_scale, stream=None, check=True):
    """Scatters pages from `outer_mem` back into the cache and its scales (the inverse of kv_cache_reorder)."""
    s, d = _lib.ReorderStride.of(src_stride), _lib.ReorderStride.of(dst_stride)
    rc = _lib.lib().pmxhip_kv_cache_invert_reorder(_stream(stream), _ptr(outer_mem), _ptr(page_ids), ctypes.byref(s),
                                                   ctypes.byref(d), int(page_ids.numel()), layers, kv_heads, tokens,
                                                   head_dim, group_size, tp_rank, tp_size, _ptr(kv_cache), _ptr(kv_scale))
    if check and rc != RC_SUCCESS:
        raise PmxError(rc, "kv_cache_invert_reorder")
    return rc


LINEAR_VENDOR_GEMM = 1  # PMXHIP_LINEAR_VENDOR_GEMM


def row_parallel_linear_workspace_size(m, in_features, out_features, vendor_gemm=False):
    """Bytes of workspace that let row_parallel_linear split the k range over the CUs (0 = none needed); with
    `vendor_gemm`, what the vendor library is offered from 384 rows on."""
    return int(_lib.lib().pmxhip_row_parallel_linear_workspace_size_ex(m, in_features, out_features,
                                                                        LINEAR_VENDOR_GEMM if vendor_gemm else 0))


def vendor_gemm_available():
    """True when hipBLASLt could be loaded and gave a handle on the current device (allocates; never under capture)."""
    return _lib.lib().pmxhip_init_vendor_gemm() == RC_SUCCESS


def row_parallel_linear(input, weight, bias, output, *, workspace=None, stream=None, check=True, vendor_gemm=False):
    """output (M, N) = input (M, K) @ weight (N, K)^T + bias (N) or None; fp16 tensors, rows contiguous along their
    last dimension (row strides may exceed the row).  The single-rank case of the reference's row_parallel_linear.
    `workspace`: a uint8 tensor of row_parallel_linear_workspace_size bytes, or None (slower at decode sizes).
    `vendor_gemm`: from 384 rows on, hand the GEMM to hipBLASLt where it loads (off: this library's kernels)."""
    n, k = int(weight.shape[0]), int(weight.shape[1])
    m = input.numel() // k  # a contiguous (B, Hq, D) attention output is the (B, Hq * D) input in place

    def row_stride(t, width):
        if t.is_contiguous():
            return width
        if t.dim() != 2 or t.stride(1) != 1:
            raise ValueError("a tensor with padded rows must be 2-d with unit stride along the row")
        return int(t.stride(0))
    rc = _lib.lib().pmxhip_row_parallel_linear_ex(_stream(stream), _ptr(input), _ptr(weight), _ptr(bias), m, k, n,
                                                  row_stride(input, k), row_stride(weight, k), row_stride(output, n),
                                                  0 if workspace is None else workspace.numel() * workspace.element_size(),
                                                  _ptr(workspace), _ptr(output), LINEAR_VENDOR_GEMM if vendor_gemm else 0)
    if check and rc != RC_SUCCESS:
        raise PmxError(rc, "row_parallel_linear")
    return rc


class DynamicBatchingMultiHeadCacheAttention:
    """The operator class (C++ `dynamic_batching_multi_head_cache_attention`) behind its C handle."""

    def __init__(self):
        self._h = _lib.lib().pmxhip_mhca_create()
        if not self._h:
            raise MemoryError("pmxhip_mhca_create failed")
        self._keep = None
        self.workspace = None

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h and _lib is not None and _lib._lib is not None:  # module globals are gone at interpreter exit
            _lib._lib.pmxhip_mhca_destroy(h)

    def heuristic_prepare(self, *, query=None, query_shape, current_key=None, current_key_shape,
                          current_value=None, current_value_shape, attn_mask=None, attn_mask_shape=(),
                          seqstarts=None, kvstarts=None, cachestarts=None, start_pos=None, alibi_slopes=None,
                          is_causal=True, batch, decoding_batches, max_seqlen, max_kvlen, layer_idx, num_layer,
                          num_heads, num_kv_heads, head_dim, cache_mode, page_size, cache_stride_s,
                          cache_stride_l, cache_stride_h, cache_stride_kv, cachestarts_stride_b,
                          enable_cache_prefill=True, enable_sharemem_mhca=True, enable_infinity_mhca=True,
                          enable_infinity_gqca=True, specify_decoding_multi_block=1, specify_decoding_tpb=0,
                          cache=None, scale=None, output=None, output_shape, datatype=DATATYPE_FLOAT16,
                          compute_units_override=None, shared_mem_per_block_optin=65536):
        """Same arguments, in the same order of meaning, as the reference's heuristic_prepare
        (multi_head_cache_attention.h:107-148).  Returns the status code; pointers may be None
        for host-only validation runs."""
        a = MhcaPrepareArgs()
        a.compute_units = compute_units_override if compute_units_override is not None else compute_units()
        a.shared_mem_per_block_optin = shared_mem_per_block_optin
        a.query_shape = TensorShape.of(query_shape, datatype)
        a.query = _ptr(query)
        a.current_key_shape = TensorShape.of(current_key_shape, datatype)
        a.current_key = _ptr(current_key)
        a.current_value_shape = TensorShape.of(current_value_shape, datatype)
        a.current_value = _ptr(current_value)
        a.attn_mask_shape = TensorShape.of(attn_mask_shape, datatype)
        a.attn_mask = _ptr(attn_mask)
        a.seqstarts = _ptr(seqstarts)
        a.kvstarts = _ptr(kvstarts)
        a.cachestarts = _ptr(cachestarts)
        a.start_pos = _ptr(start_pos)
        a.alibi_slopes = _ptr(alibi_slopes)
        a.is_causal = 1 if is_causal else 0
        a.batch = batch
        a.decoding_batches = decoding_batches
        a.max_seqlen = max_seqlen
        a.max_kvlen = max_kvlen
        a.layer_idx = layer_idx
        a.num_layer = num_layer
        a.num_heads = num_heads
        a.num_kv_heads = num_kv_heads
        a.head_dim = head_dim
        a.cache_mode = cache_mode
        a.page_size = page_size
        a.cache_stride_s = cache_stride_s
        a.cache_stride_l = cache_stride_l
        a.cache_stride_h = cache_stride_h
        a.cache_stride_kv = cache_stride_kv
        a.cachestarts_stride_b = cachestarts_stride_b
        a.enable_cache_prefill = int(enable_cache_prefill)
        a.enable_sharemem_mhca = int(enable_sharemem_mhca)
        a.enable_infinity_mhca = int(enable_infinity_mhca)
        a.enable_infinity_gqca = int(enable_infinity_gqca)
        a.specify_decoding_multi_block = specify_decoding_multi_block
        a.specify_decoding_tpb = specify_decoding_tpb
        a.cache = _ptr(cache)
        a.scale = _ptr(scale)
        a.output_shape = TensorShape.of(output_shape, datatype)
        a.output = _ptr(output)
        # keep the tensors alive for as long as the operator may launch on them
        self._keep = (query, current_key, current_value, attn_mask, seqstarts, kvstarts, cachestarts, start_pos,
                      alibi_slopes, cache, scale, output)
        return _lib.lib().pmxhip_mhca_heuristic_prepare(self._h, ctypes.byref(a))

    @property
    def cfg(self):
        d = MhcaDerived()
        rc = _lib.lib().pmxhip_mhca_get_derived(self._h, ctypes.byref(d))
        if rc != RC_SUCCESS:
            raise PmxError(rc, "cfg (heuristic_prepare has not succeeded)")
        return d

    def set_workspace(self, workspace):
        self.workspace = workspace
        return _lib.lib().pmxhip_mhca_set_workspace(self._h, _ptr(workspace))

    def allocate_workspace(self, device="cuda"):
        n = int(self.cfg.workspace_size)
        ws = torch.empty(max(n, 16), dtype=torch.uint8, device=device) if n > 0 else None
        self.set_workspace(ws)
        return ws

    def forward_kvstore(self, stream=None):
        return _lib.lib().pmxhip_mhca_forward_kvstore(self._h, _stream(stream))

    def forward_decode(self, stream=None):
        return _lib.lib().pmxhip_mhca_forward_decode(self._h, _stream(stream))

    def forward_prefill(self, stream=None):
        return _lib.lib().pmxhip_mhca_forward_prefill(self._h, _stream(stream))

    def forward(self, stream=None):
        return _lib.lib().pmxhip_mhca_forward(self._h, _stream(stream))

    def forward_streams(self, stream, side_stream, fork_event, join_event):
        """forward() of a mixed step with the decode stage on `side_stream` beside the prefill stage on `stream`;
        the two torch.cuda.Event objects are the fork and the join (recorded once before, so that they exist)."""
        return _lib.lib().pmxhip_mhca_forward_streams(self._h, _stream(stream), _stream(side_stream),
                                                      ctypes.c_void_p(fork_event.cuda_event),
                                                      ctypes.c_void_p(join_event.cuda_event))
