"""ctypes binding of the C ABI declared in include/pmx_hip/c_api.h.

The library is loaded from this directory only.  There is no fallback: if
libpmx_hip.so is absent the import of any operator raises."""
import ctypes
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libpmx_hip.so")

c_i64 = ctypes.c_int64
c_i32 = ctypes.c_int32
c_f32 = ctypes.c_float
c_vp = ctypes.c_void_p

PMXHIP_SUCCESS = 0
PMXHIP_OTHER_ERROR = 1
PMXHIP_UNSUPPORTED = 2
PMXHIP_INVALID_VALUE = 4
DATATYPE_FLOAT16 = 5
DATATYPE_FLOAT32 = 6

EXPORTED_SYMBOLS = (
    "pmxhip_version", "pmxhip_last_error",
    "pmxhip_kv_cache_quantize", "pmxhip_key_value_cache",
    "pmxhip_init",
    "pmxhip_decode_plan_make", "pmxhip_decode_plan_make_kernel", "pmxhip_decode_attention",
    "pmxhip_decode_attention_stage", "pmxhip_decode_attention_static", "pmxhip_decode_kernel_name",
    "pmxhip_splitkv_combine",
    "pmxhip_prefill_attention", "pmxhip_prefill_workspace_size",
    "pmxhip_mhca_create", "pmxhip_mhca_destroy", "pmxhip_mhca_heuristic_prepare",
    "pmxhip_mhca_get_derived", "pmxhip_mhca_set_workspace",
    "pmxhip_mhca_forward_kvstore", "pmxhip_mhca_forward_decode", "pmxhip_mhca_forward_prefill",
    "pmxhip_mhca_forward", "pmxhip_mhca_forward_streams",
    "pmxhip_kv_cache_reorder", "pmxhip_kv_cache_invert_reorder",
    "pmxhip_rotary_position_embedding", "pmxhip_rope_kv_cache_quantize",
    "pmxhip_row_parallel_linear", "pmxhip_row_parallel_linear_workspace_size",
    "pmxhip_row_parallel_linear_ex", "pmxhip_row_parallel_linear_workspace_size_ex", "pmxhip_init_vendor_gemm",
)


class KvstoreParams(ctypes.Structure):
    _fields_ = [
        ("current_key", c_vp), ("current_value", c_vp),
        ("seqstarts", c_vp), ("cachestarts", c_vp), ("start_pos", c_vp),
        ("num_layer", c_i64), ("layer_idx", c_i64), ("num_kv_heads", c_i64), ("head_dim", c_i64),
        ("page_size", c_i32),
        ("current_key_stride_s", c_i64), ("current_value_stride_s", c_i64),
        ("cache_stride_s", c_i64), ("cache_stride_l", c_i64), ("cache_stride_h", c_i64),
        ("cache_stride_kv", c_i64), ("cachestarts_stride_b", c_i64),
        ("cache", c_vp), ("scale", c_vp),
        ("batch", c_i64), ("max_seqlen", c_i64), ("cache_mode", c_i32),
    ]


class DecodeParams(ctypes.Structure):
    _fields_ = [
        ("query", c_vp), ("attn_mask", c_vp), ("output", c_vp), ("cache", c_vp), ("scale", c_vp),
        ("cachestarts", c_vp), ("kvstarts", c_vp),
        ("attn_scale", c_f32),
        ("layer_idx", c_i64), ("num_kv_repeats", c_i64), ("page_size", c_i64),
        ("query_stride_s", c_i64), ("output_stride_s", c_i64),
        ("mask_stride_s", c_i64), ("mask_stride_h", c_i64),
        ("cache_stride_s", c_i64), ("cache_stride_l", c_i64), ("cache_stride_h", c_i64),
        ("cache_stride_kv", c_i64), ("cachestarts_stride_b", c_i64),
        ("decoding_batches", c_i64), ("num_heads", c_i64), ("num_kv_heads", c_i64), ("head_dim", c_i64),
        ("cache_mode", c_i32), ("num_token_ranges", c_i32),
        ("workspace", c_vp), ("workspace_size", c_i64),
        ("kernel_request", c_i32),
    ]


class DecodePlan(ctypes.Structure):
    _fields_ = [
        ("num_token_ranges", c_i32), ("kv_heads_per_group", c_i32),
        ("q_heads_per_pass", c_i32), ("num_passes", c_i32),
        ("partial_out_size", c_i64), ("partial_ml_size", c_i64), ("workspace_size", c_i64),
        ("kernel", c_i32),
    ]


# pmxhip_decode_kernel_t
DECODE_KERNEL_AUTO = 0
DECODE_KERNEL_GENERAL = 1
DECODE_KERNEL_QUAD = 2
DECODE_KERNEL_MFMA16 = 3
DECODE_KERNEL_MFMA32 = 4
STATIC_WORKSPACE_BYTES = 32 * 1024 * 1024


class PrefillParams(ctypes.Structure):
    _fields_ = [
        ("query", c_vp), ("output", c_vp), ("cache", c_vp), ("scale", c_vp),
        ("seqstarts", c_vp), ("kvstarts", c_vp), ("cachestarts", c_vp),
        ("attn_scale", c_f32), ("is_causal", c_i32),
        ("batch", c_i64), ("decoding_batches", c_i64), ("max_seqlen", c_i64), ("max_kvlen", c_i64),
        ("layer_idx", c_i64), ("num_heads", c_i64), ("num_kv_heads", c_i64), ("head_dim", c_i64),
        ("cache_mode", c_i32), ("page_size", c_i64),
        ("query_stride_s", c_i64), ("output_stride_s", c_i64),
        ("cache_stride_s", c_i64), ("cache_stride_l", c_i64), ("cache_stride_h", c_i64),
        ("cache_stride_kv", c_i64), ("cachestarts_stride_b", c_i64),
        ("attn_mask", c_vp), ("mask_stride_s", c_i64), ("mask_stride_h", c_i64), ("alibi_slopes", c_vp),
        ("current_key", c_vp), ("current_value", c_vp), ("key_stride_s", c_i64), ("value_stride_s", c_i64),
        ("prefill_query_rows", c_i64),
        ("workspace", c_vp), ("workspace_size", c_i64),
    ]


class RopeParams(ctypes.Structure):
    _fields_ = [
        ("query", c_vp), ("key", c_vp), ("start_pos", c_vp), ("seqstarts", c_vp),
        ("theta", c_f32), ("bypass_key", c_i32), ("rotary_dim", c_i64), ("batch", c_i64),
        ("num_heads", c_i64), ("num_key_heads", c_i64), ("head_dim", c_i64), ("max_seqlen", c_i64),
        ("max_position_embeddings", c_i64), ("scaling_type", c_i32), ("scaling_factor", c_f32),
        ("query_stride_s", c_i64), ("key_stride_s", c_i64), ("rotated_query_stride_s", c_i64),
        ("rotated_key_stride_s", c_i64), ("rotated_query", c_vp), ("rotated_key", c_vp),
    ]


class ReorderStride(ctypes.Structure):
    """pmxhip_reorder_stride: byte strides {page, layer, plane, head, token, byte} of the cache, then of the scales."""
    _fields_ = [(n + k, c_i32) for k in ("_cache", "_scale")
                for n in ("p_stride", "l_stride", "kv_stride", "h_stride", "t_stride", "d_stride")]

    @staticmethod
    def of(values):
        s = ReorderStride()
        for (name, _), v in zip(ReorderStride._fields_, values):
            setattr(s, name, int(v))
        return s


class TensorShape(ctypes.Structure):
    _fields_ = [("dim_count", c_i32), ("data_type", c_i32), ("dims", c_i64 * 4)]

    @staticmethod
    def of(dims, data_type=DATATYPE_FLOAT16):
        s = TensorShape()
        s.dim_count = len(dims)
        s.data_type = data_type
        for i, d in enumerate(dims):
            s.dims[i] = int(d)
        return s


class MhcaPrepareArgs(ctypes.Structure):
    _fields_ = [
        ("compute_units", c_i32), ("shared_mem_per_block_optin", c_i64),
        ("query_shape", TensorShape), ("query", c_vp),
        ("current_key_shape", TensorShape), ("current_key", c_vp),
        ("current_value_shape", TensorShape), ("current_value", c_vp),
        ("attn_mask_shape", TensorShape), ("attn_mask", c_vp),
        ("seqstarts", c_vp), ("kvstarts", c_vp), ("cachestarts", c_vp), ("start_pos", c_vp),
        ("alibi_slopes", c_vp),
        ("is_causal", c_i32),
        ("batch", c_i64), ("decoding_batches", c_i64), ("max_seqlen", c_i64), ("max_kvlen", c_i64),
        ("layer_idx", c_i64), ("num_layer", c_i64),
        ("num_heads", c_i64), ("num_kv_heads", c_i64), ("head_dim", c_i64),
        ("cache_mode", c_i32), ("page_size", c_i64),
        ("cache_stride_s", c_i64), ("cache_stride_l", c_i64), ("cache_stride_h", c_i64),
        ("cache_stride_kv", c_i64), ("cachestarts_stride_b", c_i64),
        ("enable_cache_prefill", c_i32), ("enable_sharemem_mhca", c_i32),
        ("enable_infinity_mhca", c_i32), ("enable_infinity_gqca", c_i32),
        ("specify_decoding_multi_block", c_i32), ("specify_decoding_tpb", c_i32),
        ("cache", c_vp), ("scale", c_vp),
        ("output_shape", TensorShape), ("output", c_vp),
    ]


class MhcaDerived(ctypes.Structure):
    _fields_ = [
        ("prefill_batches", c_i64),
        ("q_stride_s", c_i64), ("k_stride_s", c_i64), ("v_stride_s", c_i64), ("o_stride_s", c_i64),
        ("mask_stride_s", c_i64), ("mask_stride_h", c_i64),
        ("attn_scale", c_f32),
        ("num_kv_repeats", c_i64),
        ("decoding_algo", c_i32),
        ("decoding_threads_per_block", c_i64), ("decoding_multi_block_size", c_i64),
        ("decoding_multi_block_partial_out_size", c_i64),
        ("decoding_multi_block_partial_log_sum_exp_size", c_i64),
        ("decoding_multi_block_counter_size", c_i64),
        ("workspace_size", c_i64),
    ]


_lib = None


def lib():
    """The loaded library.  Raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            "libpmx_hip.so is missing at %s: build it with __graft_entry__.build() "
            "(there is no CPU or PyTorch fallback)" % LIB_PATH)
    L = ctypes.CDLL(LIB_PATH)
    L.pmxhip_version.restype = ctypes.c_char_p
    L.pmxhip_last_error.restype = ctypes.c_char_p
    L.pmxhip_kv_cache_quantize.restype = ctypes.c_int
    L.pmxhip_kv_cache_quantize.argtypes = [ctypes.POINTER(KvstoreParams), c_vp]
    L.pmxhip_rotary_position_embedding.restype = ctypes.c_int
    L.pmxhip_rotary_position_embedding.argtypes = [ctypes.POINTER(RopeParams), c_vp]
    L.pmxhip_rope_kv_cache_quantize.restype = ctypes.c_int
    L.pmxhip_rope_kv_cache_quantize.argtypes = [ctypes.POINTER(RopeParams), ctypes.POINTER(KvstoreParams), c_vp]
    L.pmxhip_kv_cache_reorder.restype = ctypes.c_int
    L.pmxhip_kv_cache_reorder.argtypes = [c_vp] * 4 + [ctypes.POINTER(ReorderStride)] * 2 + [c_i64] * 8 + [c_vp]
    L.pmxhip_kv_cache_invert_reorder.restype = ctypes.c_int
    L.pmxhip_kv_cache_invert_reorder.argtypes = [c_vp] * 3 + [ctypes.POINTER(ReorderStride)] * 2 + [c_i64] * 8 + [c_vp] * 2
    L.pmxhip_key_value_cache.restype = ctypes.c_int
    L.pmxhip_key_value_cache.argtypes = [c_vp] * 6 + [c_i64] * 6 + [c_i32] + [c_i64] * 6 + [c_vp] * 2
    L.pmxhip_decode_plan_make.restype = ctypes.c_int
    L.pmxhip_decode_plan_make.argtypes = [c_i64] * 5 + [c_i32, c_i32, ctypes.POINTER(DecodePlan)]
    L.pmxhip_row_parallel_linear.restype = ctypes.c_int
    L.pmxhip_row_parallel_linear.argtypes = [c_vp] * 4 + [c_i64] * 7 + [c_vp, c_vp]
    L.pmxhip_row_parallel_linear_workspace_size.restype = c_i64
    L.pmxhip_row_parallel_linear_workspace_size.argtypes = [c_i64] * 3
    L.pmxhip_row_parallel_linear_ex.restype = ctypes.c_int
    L.pmxhip_row_parallel_linear_ex.argtypes = [c_vp] * 4 + [c_i64] * 7 + [c_vp, c_vp, ctypes.c_int32]
    L.pmxhip_row_parallel_linear_workspace_size_ex.restype = c_i64
    L.pmxhip_row_parallel_linear_workspace_size_ex.argtypes = [c_i64] * 3 + [ctypes.c_int32]
    L.pmxhip_init_vendor_gemm.restype = ctypes.c_int
    L.pmxhip_init_vendor_gemm.argtypes = []
    L.pmxhip_init.restype = ctypes.c_int
    L.pmxhip_init.argtypes = []
    L.pmxhip_decode_plan_make_kernel.restype = ctypes.c_int
    L.pmxhip_decode_plan_make_kernel.argtypes = [c_i64] * 5 + [c_i32, c_i32, c_i32, ctypes.POINTER(DecodePlan)]
    L.pmxhip_decode_attention_static.restype = ctypes.c_int
    L.pmxhip_decode_attention_static.argtypes = [ctypes.POINTER(DecodeParams), c_vp]
    L.pmxhip_decode_kernel_name.restype = ctypes.c_char_p
    L.pmxhip_decode_kernel_name.argtypes = [ctypes.POINTER(DecodeParams)]
    L.pmxhip_decode_attention.restype = ctypes.c_int
    L.pmxhip_decode_attention.argtypes = [ctypes.POINTER(DecodeParams), c_vp]
    L.pmxhip_decode_attention_stage.restype = ctypes.c_int
    L.pmxhip_decode_attention_stage.argtypes = [ctypes.POINTER(DecodeParams), c_i32, c_vp]
    L.pmxhip_splitkv_combine.restype = ctypes.c_int
    L.pmxhip_splitkv_combine.argtypes = [c_vp] * 4 + [c_i64, c_i64, c_vp, c_vp]
    L.pmxhip_prefill_workspace_size.restype = c_i64
    L.pmxhip_prefill_workspace_size.argtypes = [c_i64] * 7 + [c_i32]
    L.pmxhip_prefill_attention.restype = ctypes.c_int
    L.pmxhip_prefill_attention.argtypes = [ctypes.POINTER(PrefillParams), c_vp]
    L.pmxhip_mhca_create.restype = c_vp
    L.pmxhip_mhca_create.argtypes = []
    L.pmxhip_mhca_destroy.restype = None
    L.pmxhip_mhca_destroy.argtypes = [c_vp]
    L.pmxhip_mhca_heuristic_prepare.restype = ctypes.c_int
    L.pmxhip_mhca_heuristic_prepare.argtypes = [c_vp, ctypes.POINTER(MhcaPrepareArgs)]
    L.pmxhip_mhca_get_derived.restype = ctypes.c_int
    L.pmxhip_mhca_get_derived.argtypes = [c_vp, ctypes.POINTER(MhcaDerived)]
    L.pmxhip_mhca_set_workspace.restype = ctypes.c_int
    L.pmxhip_mhca_set_workspace.argtypes = [c_vp, c_vp]
    for name in ("pmxhip_mhca_forward_kvstore", "pmxhip_mhca_forward_decode",
                 "pmxhip_mhca_forward_prefill", "pmxhip_mhca_forward"):
        fn = getattr(L, name)
        fn.restype = ctypes.c_int
        fn.argtypes = [c_vp, c_vp]
    L.pmxhip_mhca_forward_streams.restype = ctypes.c_int
    L.pmxhip_mhca_forward_streams.argtypes = [c_vp] * 5
    _lib = L
    return L


def last_error():
    return lib().pmxhip_last_error().decode()
