/*
 * C ABI of the MI355X (gfx950) int8-KV dynamic-batching attention path.
 *
 * The reference library has no C ABI: its boundary is the C++ class
 * ppl::kernel::llm::cuda::pmx::dynamic_batching_multi_head_cache_attention
 * (include/ppl/kernel/llm/cuda/pmx/multi_head_cache_attention.h:25-159).  The
 * entry points below are what that class bottoms out in -- one per kernel launch
 * site of src/ppl/kernel/llm/cuda/pmx/multi_head_cache_attention/kernel.cu -- with
 * plain pointers and sizes only, so that any FFI can bind them.  The C++ class in
 * cache_attention.h (this directory) marshals its cfg into these.
 *
 * Conventions shared by every entry point:
 *   - all pointers are device pointers unless stated otherwise; the caller owns
 *     every buffer; nothing is allocated, freed or synchronised by the library;
 *   - work is enqueued on `stream` (a hipStream_t; NULL = the null stream);
 *   - half tensors are IEEE binary16; index arrays are int64;
 *   - cache element (token t, layer l, K/V plane kv, kv head h, channel d) lives at
 *       t*cache_stride_s + l*cache_stride_l + kv*cache_stride_kv + h*cache_stride_h + d
 *     in the int8 cache, and its group-of-8 scale at that index / 8 in the scale
 *     tensor (kernel.cu:117-126); all four strides must be multiples of 8;
 *   - cache_mode 0: token t of sequence b is row cachestarts[b] + t;
 *     cache_mode 1: row cachestarts[b*cachestarts_stride_b + t/128] + t%128
 *     (kernel.cu:97-100, 365-368);
 *   - return value: a pmxhip_status_t (0 = success).
 */
#ifndef PMX_HIP_C_API_H_
#define PMX_HIP_C_API_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#if defined(__GNUC__)
#define PMXHIP_API __attribute__((visibility("default")))
#else
#define PMXHIP_API
#endif

/* Same numeric values as ppl::common::RetCode (ppl.common retcode.h, not part of
 * the reference tree; only these four are used on this path). */
typedef enum pmxhip_status_t {
    PMXHIP_SUCCESS = 0,
    PMXHIP_OTHER_ERROR = 1,
    PMXHIP_UNSUPPORTED = 2,
    PMXHIP_INVALID_VALUE = 4
} pmxhip_status_t;

typedef struct ihipStream_t* pmxhip_stream_t; /* == hipStream_t */

#define PMXHIP_PAGE_SIZE 128 /* UNIFORM_PAGE_SIZE, kernel.cu:31 */

/* ---- quantise/append ------------------------------------------------------
 * Replaces dynamic_batching_kv_cache_quantize_kernel_param (kernel.cu:64-84) and
 * the launch in forward_kvstore (kernel.cu:2013-2057).  Fields up to `scale` are
 * the reference's, in the reference's order; the rest are what the launch site
 * reads from cfg. */
typedef struct pmxhip_kvstore_params {
    const void* current_key;   /* half (S, KVH, D) */
    const void* current_value; /* half (S, KVH, D) */
    const int64_t* seqstarts;  /* (B + 1) */
    const int64_t* cachestarts; /* (B) or (B, MaxP) */
    const int64_t* start_pos;  /* (B) */
    int64_t num_layer;
    int64_t layer_idx;
    int64_t num_kv_heads;
    int64_t head_dim;
    int32_t page_size; /* used when cache_mode == 1; must be 128 */
    int64_t current_key_stride_s;
    int64_t current_value_stride_s;
    int64_t cache_stride_s;
    int64_t cache_stride_l;
    int64_t cache_stride_h;
    int64_t cache_stride_kv;
    int64_t cachestarts_stride_b;
    void* cache; /* int8 */
    void* scale; /* half */
    /* launch-site values (cfg.batch, cfg.max_seqlen, cfg.cache_mode) */
    int64_t batch;
    int64_t max_seqlen; /* upper bound of seqstarts[b+1]-seqstarts[b] */
    int32_t cache_mode; /* 0 contiguous, 1 paged */
} pmxhip_kvstore_params;

PMXHIP_API int pmxhip_kv_cache_quantize(const pmxhip_kvstore_params* p, pmxhip_stream_t stream);

/* ---- decode attention (one query token per sequence) -----------------------
 * Replaces dynamic_batching_decoding_cache_attention_kernel_param
 * (kernel.cu:35-62) and forward_decode (kernel.cu:2059-2125), including the
 * split-KV partials and their combine (kernel.cu:600-678).  The split is not a
 * fixed block count: the kv tokens of all decode sequences form one stream that
 * is cut into `num_token_ranges` equal ranges, one workgroup each, and a second
 * kernel merges the pieces of every sequence that spans more than one range.
 * Zero the struct before filling it in (memset, `= {0}`): fields added behind the
 * reference's, such as kernel_request, mean "as before" only when they are zero.
 *
 * Cache layout: the four strides are free (any order of layer, K/V plane, token and
 * kv head, multiples of 16 bytes).  A kernel addresses a row as a 64-bit base per
 * wave plus a 32-bit offset per lane, so what must lie within 2 GiB is one block of
 * tokens of one kv head: 32 * cache_stride_s + head_dim < 2^31 always suffices
 * (prefill: 64 * cache_stride_s + head_dim).  cache_stride_h may be anything: where
 * two neighbouring kv heads lie 2 GiB or more apart (a (L, KVH, S, 2, D) pool of
 * more than 2^23 tokens at head_dim 128) a kernel with a wave per kv head runs the
 * step instead of the quad kernel, and only an explicit kernel_request for the quad
 * kernel is refused (PMXHIP_UNSUPPORTED). */
typedef struct pmxhip_decode_params {
    const void* query;     /* half (B_dec, Hq, D); row = sequence index */
    const void* attn_mask; /* half, optional (NULL = none) */
    void* output;          /* half (B_dec, Hq, D) */
    const void* cache;     /* int8 */
    const void* scale;     /* half */
    const int64_t* cachestarts;
    const int64_t* kvstarts; /* (B_dec + 1) */
    float attn_scale;
    int64_t layer_idx;
    int64_t num_kv_repeats; /* Hq / KVH */
    int64_t page_size;
    int64_t query_stride_s;
    int64_t output_stride_s;
    int64_t mask_stride_s;
    int64_t mask_stride_h;
    int64_t cache_stride_s;
    int64_t cache_stride_l;
    int64_t cache_stride_h;
    int64_t cache_stride_kv;
    int64_t cachestarts_stride_b;
    /* launch-site values */
    int64_t decoding_batches;
    int64_t num_heads;
    int64_t num_kv_heads;
    int64_t head_dim;
    int32_t cache_mode;
    /* split-KV plan: from pmxhip_decode_plan_make(); workspace >= plan.workspace_size */
    int32_t num_token_ranges;
    void* workspace;
    int64_t workspace_size;
    /* 0 (PMXHIP_DECODE_KERNEL_AUTO) = the library chooses the token-range kernel by shape.  Any other
     * pmxhip_decode_kernel_t insists on that kernel (comparison runs, tests of every kernel on one shape); the
     * call fails with PMXHIP_UNSUPPORTED when that kernel does not serve the shape or the buffers.  The plan
     * must have been made for the same request (pmxhip_decode_plan_make_kernel). */
    int32_t kernel_request;
} pmxhip_decode_params;

/* The token-range kernels of the decode step.  The reference chooses among its three kernels with the
 * enable_* flags of heuristic_prepare (utils.cu:136-264); here the choice follows from the shape. */
typedef enum pmxhip_decode_kernel_t {
    PMXHIP_DECODE_KERNEL_AUTO = 0,
    PMXHIP_DECODE_KERNEL_GENERAL = 1, /* VALU; every head_dim and head count */
    PMXHIP_DECODE_KERNEL_QUAD = 2,    /* head_dim 64 or 128 (two or more kv heads) or 256, up to 4 query heads per
                                         kv head (8 at head_dim 256, and at head_dim 128 with kv heads in eights) */
    PMXHIP_DECODE_KERNEL_MFMA16 = 3,  /* head_dim 128, up to 16 query heads per kv head as MFMA columns */
    PMXHIP_DECODE_KERNEL_MFMA32 = 4   /* head_dim 128 or 64, 32 columns; more query heads per kv head in passes of 32 */
} pmxhip_decode_kernel_t;

typedef struct pmxhip_decode_plan {
    int32_t num_token_ranges;   /* workgroups along the kv-token stream */
    int32_t kv_heads_per_group; /* kv heads one workgroup serves */
    int32_t q_heads_per_pass;   /* query heads per kv head served at once: 1, 2, 4 or 8 from registers (general
                                   and quad kernels), or the 16 / 32 MFMA columns */
    int32_t num_passes;         /* ceil(num_kv_repeats / q_heads_per_pass) */
    int64_t partial_out_size;   /* bytes: float32 partial outputs */
    int64_t partial_ml_size;    /* bytes: float32 (running max, exp-sum) pairs */
    int64_t workspace_size;     /* total bytes */
    int32_t kernel;             /* pmxhip_decode_kernel_t the plan was made for.  The launch falls back to the
                                   general kernel when the quad kernel's needs of the buffers (16-byte aligned
                                   output rows) are not met; pmxhip_decode_kernel_name tells what a call runs. */
} pmxhip_decode_plan;

/* Host-only.  `compute_units` is hipDeviceProp_t::multiProcessorCount (0 = ask the current device).
 * `num_token_ranges_hint` 0 = choose; > 0 = use exactly this many ranges. */
PMXHIP_API int pmxhip_decode_plan_make(int64_t decoding_batches, int64_t num_heads, int64_t num_kv_heads,
                                       int64_t head_dim, int64_t max_kvlen, int32_t compute_units,
                                       int32_t num_token_ranges_hint, pmxhip_decode_plan* plan);
/* The same for a requested kernel (pmxhip_decode_params::kernel_request). */
PMXHIP_API int pmxhip_decode_plan_make_kernel(int64_t decoding_batches, int64_t num_heads, int64_t num_kv_heads,
                                              int64_t head_dim, int64_t max_kvlen, int32_t compute_units,
                                              int32_t num_token_ranges_hint, int32_t kernel_request,
                                              pmxhip_decode_plan* plan);

PMXHIP_API int pmxhip_decode_attention(const pmxhip_decode_params* p, pmxhip_stream_t stream);

/* Name of the token-range kernel that pmxhip_decode_attention(p) launches ("" if the call would be rejected):
 * one of decode_attention_kernel, decode_attention_quad_kernel, decode_attention_mfma16_kernel,
 * decode_attention_mfma_kernel -- the names a profiler's kernel trace shows.  Host only, launches nothing. */
PMXHIP_API const char* pmxhip_decode_kernel_name(const pmxhip_decode_params* p);

/* pmxhip_decode_attention for callers that cannot allocate: it has no counterpart in the reference, whose caller
 * always sizes and passes cfg.workspace (multi_head_cache_attention.h:104-106).  It is for code that must not
 * call hipMalloc -- a step recorded under HIP graph capture, a serving loop or harness that forbids allocation:
 * p->workspace and p->workspace_size are ignored and the split-KV pieces go to a static array of
 * PMXHIP_STATIC_WORKSPACE_BYTES inside the library (one per GPU, held until the process ends).  The call
 * allocates and frees nothing.  A step whose pieces need more -- (num_token_ranges + decoding_batches) *
 * num_heads * (head_dim + 2) * 4 bytes -- is rejected with PMXHIP_INVALID_VALUE.  All calls on one GPU share the
 * array: calls that overlap on one GPU (two streams, two threads) race; calls on one stream are safe.  Nothing in
 * the array needs clearing between calls: a piece is read back only by the step that wrote it.  The first call
 * on a device resolves the array's address (hipGetSymbolAddress); under stream capture do that beforehand with
 * pmxhip_init(). */
#define PMXHIP_STATIC_WORKSPACE_BYTES (32 * 1024 * 1024)
PMXHIP_API int pmxhip_decode_attention_static(const pmxhip_decode_params* p, pmxhip_stream_t stream);

/* The same step split at its kernel boundary, for callers that time or overlap
 * the two kernels: stage 1 = the token-range kernel only (final rows of
 * sequences that fit one range, float32 pieces of the others), stage 2 = the
 * combine kernel only, stage 0 = both (== pmxhip_decode_attention).  The
 * reference fuses the two (kernel.cu:600-678), so it has no counterpart. */
PMXHIP_API int pmxhip_decode_attention_stage(const pmxhip_decode_params* p, int32_t stage, pmxhip_stream_t stream);

/* ---- split-KV combine on caller-supplied pieces ----------------------------
 * The merge of kernel.cu:617-665 as a stand-alone kernel: for each of `rows`
 * (sequence, head) pairs, merges pieces [piece_begin[r], piece_end[r]) of
 *   partial_out float32 (pieces, D)   normalised partial outputs
 *   partial_ml  float32 (pieces, 2)   (running max in log2 units, exp-sum)
 * into output row r (half, D).  Rows with no pieces produce zeros. */
PMXHIP_API int pmxhip_splitkv_combine(const float* partial_out, const float* partial_ml,
                                      const int64_t* piece_begin, const int64_t* piece_end,
                                      int64_t rows, int64_t head_dim, void* output,
                                      pmxhip_stream_t stream);

/* ---- multi-query-token (chunked prefill) attention over the int8 cache -----
 * Replaces the flash_attn2_paged_fmha call of forward_prefill
 * (kernel.cu:2127-2179; include/ppl/kernel/llm/cuda/flash_attn2/fmha.h:73) and, with
 * current_key set, its flash_attn2_fmha call (kernel.cu:2181-2212).
 * Sequences [decoding_batches, batch) are prefill; query/output rows are
 * addressed through seqstarts, kv length through kvstarts, cache rows through
 * cachestarts; causal masking is bottom-right aligned (mask.h:186). */
typedef struct pmxhip_prefill_params {
    const void* query; /* half (S, Hq, D) */
    void* output;      /* half (S, Hq, D) */
    const void* cache;
    const void* scale;
    const int64_t* seqstarts;   /* (B + 1), whole batch */
    const int64_t* kvstarts;    /* (B + 1), whole batch */
    const int64_t* cachestarts; /* whole batch */
    float attn_scale;
    int32_t is_causal;
    int64_t batch;
    int64_t decoding_batches;
    int64_t max_seqlen;
    int64_t max_kvlen;
    int64_t layer_idx;
    int64_t num_heads;
    int64_t num_kv_heads;
    int64_t head_dim;
    int32_t cache_mode;
    int64_t page_size;
    int64_t query_stride_s;
    int64_t output_stride_s;
    int64_t cache_stride_s;
    int64_t cache_stride_l;
    int64_t cache_stride_h;
    int64_t cache_stride_kv;
    int64_t cachestarts_stride_b;
    /* Optional inputs of the two flash_attn2 calls (kernel.cu:2153-2158, 2188-2193); zero = absent.
     * attn_mask: additive half bias; element (head h, absolute query row r, absolute kv column c)
     * at h*mask_stride_h + r*mask_stride_s + c, c = kvstarts[b] + t (seqstarts[b] + t when
     * current_key is given); added to the scaled logit (flash_api.cu:171).
     * alibi_slopes: float32 (Hq); causal: + slope*t, otherwise - slope*|row + kvlen - qlen - t|
     * (flash_attn2/src/mask.h:191-197). */
    const void* attn_mask;
    int64_t mask_stride_s;
    int64_t mask_stride_h;
    const float* alibi_slopes;
    /* enable_cache_prefill = false (kernel.cu:2181-2212): with current_key != NULL the stage
     * attends over the step's own half K/V rows (S, KVH, D) only -- kv length = query length,
     * no cache read; cache/scale/cachestarts/kvstarts are then ignored. */
    const void* current_key;
    const void* current_value;
    int64_t key_stride_s;
    int64_t value_stride_s;
    /* Rows of `query` that belong to the prefill sequences; 0 = unknown.  No counterpart in the reference's
     * call, which sizes its launch from max_seqlen (kernel.cu:2143-2179); the operator class takes it from
     * the query shape that heuristic_prepare receives.  Only the launch size depends on it: the
     * batch has at most rows / (positions per workgroup) + sequences query tiles, far fewer than
     * sequences * tiles of max_seqlen when one long sequence sits among short ones. */
    int64_t prefill_query_rows;
    /* Optional workspace, NULL = none.  No counterpart in the reference's call (its flash_attn2 split-KV path keeps
     * its partial results inside the kernel's own allocation, flash_api.cu:169-178).  With at least
     * pmxhip_prefill_workspace_size() bytes (16-byte aligned) a batch of short chunks -- max_seqlen * (Hq / KVH)
     * <= 32, head_dim 64 or 128, no attn_mask, alibi or current_key -- runs on the decode step's MFMA kernels over
     * token ranges, with (query position, query head) pairs as its columns and the split-KV pieces in this
     * workspace; without it, or for any other batch, the tile kernel runs.  Results are the same within the tolerance.
     * On that path max_seqlen must bound the query rows of every prefill sequence, as it does in the reference's
     * call (kernel.cu:2143), because the step has max_seqlen query positions per sequence.  A max_seqlen that
     * prefill_query_rows proves too small (more rows than prefill sequences * max_seqlen) keeps the batch on the tile
     * kernel, which walks every row whatever the hint; otherwise the rows of a sequence beyond max_seqlen are not
     * computed and are filled with NaN, so that an understated hint shows in the output.  A layout or alignment that
     * the decode kernels refuse also keeps the batch on the tile kernel. */
    void* workspace;
    int64_t workspace_size;
} pmxhip_prefill_params;

PMXHIP_API int pmxhip_prefill_attention(const pmxhip_prefill_params* p, pmxhip_stream_t stream);

/* Bytes of pmxhip_prefill_params::workspace with which a batch runs its short chunks on the decode step's kernel;
 * 0 when the batch is not one of short chunks (the tile kernel needs no workspace).  compute_units 0 = those of the
 * current device.  The operator class adds this to what it reports as cfg.workspace_size (the decode and the
 * prefill stage run one after the other on the stream and share the buffer). */
PMXHIP_API int64_t pmxhip_prefill_workspace_size(int64_t batch, int64_t decoding_batches, int64_t max_seqlen,
                                                 int64_t max_kvlen, int64_t num_heads, int64_t num_kv_heads,
                                                 int64_t head_dim, int32_t compute_units);

/* ---- the operator class behind a C handle -----------------------------------
 * Drives the C++ class (heuristic_prepare / forward_*) so that a non-C++ host
 * can use the reference's operator interface unchanged.  Argument meaning and
 * order follow multi_head_cache_attention.h:107-148 of the reference. */
typedef struct pmxhip_tensor_shape {
    int32_t dim_count;
    int32_t data_type; /* pmxhip DATATYPE_* value; 5 = float16 */
    int64_t dims[4];
} pmxhip_tensor_shape;

typedef struct pmxhip_mhca_prepare_args {
    int32_t compute_units;              /* device_prop.multiProcessorCount */
    int64_t shared_mem_per_block_optin; /* device_prop.sharedMemPerBlockOptin */
    pmxhip_tensor_shape query_shape;
    const void* query;
    pmxhip_tensor_shape current_key_shape;
    const void* current_key;
    pmxhip_tensor_shape current_value_shape;
    const void* current_value;
    pmxhip_tensor_shape attn_mask_shape;
    const void* attn_mask;
    const void* seqstarts;
    const void* kvstarts;
    const void* cachestarts;
    const void* start_pos;
    const void* alibi_slopes;
    int32_t is_causal;
    int64_t batch;
    int64_t decoding_batches;
    int64_t max_seqlen;
    int64_t max_kvlen;
    int64_t layer_idx;
    int64_t num_layer;
    int64_t num_heads;
    int64_t num_kv_heads;
    int64_t head_dim;
    int32_t cache_mode;
    int64_t page_size;
    int64_t cache_stride_s;
    int64_t cache_stride_l;
    int64_t cache_stride_h;
    int64_t cache_stride_kv;
    int64_t cachestarts_stride_b;
    int32_t enable_cache_prefill;
    int32_t enable_sharemem_mhca;
    int32_t enable_infinity_mhca;
    int32_t enable_infinity_gqca;
    int32_t specify_decoding_multi_block;
    int32_t specify_decoding_tpb;
    void* cache;
    void* scale;
    pmxhip_tensor_shape output_shape;
    void* output;
} pmxhip_mhca_prepare_args;

/* What heuristic_prepare derived (the "produce by prepare function" block of the
 * reference's config, multi_head_cache_attention.h:76-98). */
typedef struct pmxhip_mhca_derived {
    int64_t prefill_batches;
    int64_t q_stride_s, k_stride_s, v_stride_s, o_stride_s;
    int64_t mask_stride_s, mask_stride_h;
    float attn_scale;
    int64_t num_kv_repeats;
    int32_t decoding_algo;
    int64_t decoding_threads_per_block;
    int64_t decoding_multi_block_size;
    int64_t decoding_multi_block_partial_out_size;
    int64_t decoding_multi_block_partial_log_sum_exp_size;
    int64_t decoding_multi_block_counter_size;
    int64_t workspace_size;
} pmxhip_mhca_derived;

typedef struct pmxhip_mhca* pmxhip_mhca_t;

PMXHIP_API pmxhip_mhca_t pmxhip_mhca_create(void);
PMXHIP_API void pmxhip_mhca_destroy(pmxhip_mhca_t op);
PMXHIP_API int pmxhip_mhca_heuristic_prepare(pmxhip_mhca_t op, const pmxhip_mhca_prepare_args* args);
PMXHIP_API int pmxhip_mhca_get_derived(pmxhip_mhca_t op, pmxhip_mhca_derived* out);
PMXHIP_API int pmxhip_mhca_set_workspace(pmxhip_mhca_t op, void* workspace);
PMXHIP_API int pmxhip_mhca_forward_kvstore(pmxhip_mhca_t op, pmxhip_stream_t stream);
PMXHIP_API int pmxhip_mhca_forward_decode(pmxhip_mhca_t op, pmxhip_stream_t stream);
PMXHIP_API int pmxhip_mhca_forward_prefill(pmxhip_mhca_t op, pmxhip_stream_t stream);
PMXHIP_API int pmxhip_mhca_forward(pmxhip_mhca_t op, pmxhip_stream_t stream);
/* forward() of a mixed step with the decode stage on `side_stream`, beside the prefill stage on `stream` (they are
 * independent once the append has run): forked behind the append with `fork_event`, joined into `stream` with
 * `join_event` before the call returns.  No counterpart in the reference (multi_head_cache_attention.h:152-158 runs
 * the stages in one stream order).  Streams and events (hipEvent_t) are the caller's, of the default priority; the
 * library creates none, so the call can be captured from `stream`.  Steps that are not mixed, and steps whose two
 * attention stages share the workspace (short prefill chunks on the decode kernels), run as pmxhip_mhca_forward. */
PMXHIP_API int pmxhip_mhca_forward_streams(pmxhip_mhca_t op, pmxhip_stream_t stream, pmxhip_stream_t side_stream,
                                           void* fork_event, void* join_event);

/* ---- key_value_cache -------------------------------------------------------
 * The append step under the operator name the serving stack uses for it
 * (pmx op KeyValueCache); same arguments as pmxhip_kvstore_params, flattened.
 * In the reference tree the step is forward_kvstore (kernel.cu:2013-2057). */
PMXHIP_API int pmxhip_key_value_cache(
    pmxhip_stream_t stream,
    const void* current_key, const void* current_value,
    const int64_t* seqstarts, const int64_t* cachestarts, const int64_t* start_pos,
    int64_t batch, int64_t max_seqlen, int64_t num_layer, int64_t layer_idx,
    int64_t num_kv_heads, int64_t head_dim,
    int32_t cache_mode, int64_t page_size,
    int64_t cache_stride_s, int64_t cache_stride_l, int64_t cache_stride_h, int64_t cache_stride_kv,
    int64_t cachestarts_stride_b,
    void* cache, void* scale);

/* ---- kv_cache_reorder / kv_cache_invert_reorder ------------------------------
 * Replace ppl::kernel::llm::cuda::pmx::kv_cache_reorder and kv_cache_invert_reorder
 * (include/ppl/kernel/llm/cuda/pmx/kv_cache_reorder.h:42-74,
 * src/ppl/kernel/llm/cuda/pmx/kv_cache_reorder.cu:24-199): whole pages of the int8 cache
 * and of its scales are gathered into (scattered from) a contiguous outer buffer, for
 * swapping or migrating pages.  Both tensors are addressed as BYTES.  For slot j of
 * page_ids, layer l, plane kv in {0,1}, head h, token t < tokens and byte d:
 *   cache side:  page_ids[j]*head_dim*row + l*l_stride + kv*kv_stride + h*h_stride + t*t_stride + d*d_stride
 *                (row = head_dim for the cache, head_dim/group_size*2 for the scales; the
 *                 reference takes head_dim as the tokens of a page, kernel line 44)
 *   outer side:  (p_stride_cache + p_stride_scale)*tp_size*j + tp_rank*p_stride_cache + the five strides,
 *                scales a further (tp_size - tp_rank)*p_stride_cache + tp_rank*p_stride_scale on
 *   with p_stride_* taken from src_stride in both directions, as the reference does.
 * Field order of the stride struct is the reference's `Stride` (kv_cache_reorder.h:25-40). */
typedef struct pmxhip_reorder_stride {
    int32_t p_stride_cache, l_stride_cache, kv_stride_cache, h_stride_cache, t_stride_cache, d_stride_cache;
    int32_t p_stride_scale, l_stride_scale, kv_stride_scale, h_stride_scale, t_stride_scale, d_stride_scale;
} pmxhip_reorder_stride;

PMXHIP_API int pmxhip_kv_cache_reorder(
    pmxhip_stream_t stream, const void* kv_cache, const void* kv_scale, const int64_t* page_ids,
    const pmxhip_reorder_stride* src_stride, const pmxhip_reorder_stride* dst_stride,
    int64_t page_nums, int64_t layers, int64_t kv_heads, int64_t tokens, int64_t head_dim, int64_t group_size,
    int64_t tp_rank, int64_t tp_size, void* outer_mem);

PMXHIP_API int pmxhip_kv_cache_invert_reorder(
    pmxhip_stream_t stream, const void* outer_mem, const int64_t* page_ids,
    const pmxhip_reorder_stride* src_stride, const pmxhip_reorder_stride* dst_stride,
    int64_t page_nums, int64_t layers, int64_t kv_heads, int64_t tokens, int64_t head_dim, int64_t group_size,
    int64_t tp_rank, int64_t tp_size, void* kv_cache, void* kv_scale);

/* ---- rotary position embedding, alone and fused with the append --------------
 * pmxhip_rotary_position_embedding replaces dynamic_batching_rotary_position_embedding
 * (include/ppl/kernel/llm/cuda/pmx/rotary_position_embedding.h:54-76,
 * src/ppl/kernel/llm/cuda/pmx/rotary_position_embedding.cu:268-446): channel pairs (2i, 2i+1),
 * i < rotary_dim/2, of every query head and of the first num_key_heads key heads are rotated by
 * angle = pos / theta^(i / (rotary_dim/2)), pos = start_pos[b] + position in the sequence;
 * other channels are copied.  scaling_type: 0 none, 1 linear (pos / scaling_factor), 2 dynamic
 * (theta rescaled when start_pos + seqlen > max_position_embeddings, kernel lines 68-91); the
 * reference's header gives all three names the value 0, so only "none" is reachable there.
 * Strides are in halves per row.  rotated_query may alias query, rotated_key may alias key.
 *
 * pmxhip_rope_kv_cache_quantize is the same rotation followed, in the same kernel, by the
 * quantise/append of the rotated key and of the value rows (pmxhip_kv_cache_quantize): the
 * rotated key never makes a round trip through memory and one launch is saved.  Of `store`,
 * current_key is ignored (the key comes from `rope`); rope->rotated_key may be NULL. */
typedef struct pmxhip_rope_params {
    const void* query;         /* half (S, Hq, D) */
    const void* key;           /* half (S, KVH, D) */
    const int64_t* start_pos;  /* (B) */
    const int64_t* seqstarts;  /* (B + 1) */
    float theta;
    int32_t bypass_key;        /* 1: key rows are copied, not rotated */
    int64_t rotary_dim;
    int64_t batch;
    int64_t num_heads;
    int64_t num_key_heads;
    int64_t head_dim;
    int64_t max_seqlen;
    int64_t max_position_embeddings;
    int32_t scaling_type;
    float scaling_factor;
    int64_t query_stride_s;
    int64_t key_stride_s;
    int64_t rotated_query_stride_s;
    int64_t rotated_key_stride_s;
    void* rotated_query;
    void* rotated_key;
} pmxhip_rope_params;

PMXHIP_API int pmxhip_rotary_position_embedding(const pmxhip_rope_params* p, pmxhip_stream_t stream);
PMXHIP_API int pmxhip_rope_kv_cache_quantize(const pmxhip_rope_params* rope, const pmxhip_kvstore_params* store,
                                             pmxhip_stream_t stream);

/* ---- output projection behind the attention ---------------------------------------
 * Replaces the single-rank case of ppl::kernel::llm::cuda::pmx::row_parallel_linear
 * (include/ppl/kernel/llm/cuda/pmx/row_parallel_linear.h:28-46,
 * src/ppl/kernel/llm/cuda/pmx/row_parallel_linear.cu:25-110): output(M, N) = input(M, K) * weight(N, K)^T + bias
 * with half tensors and float32 accumulation, where the reference calls one cublasLt GEMM and, with more than
 * one rank, an all-reduce (one GPU here, so none).  The attention output (B, Hq * D) is this call's input in
 * place.  bias may be NULL.  Strides are in halves per row.  Needs N % 16 == 0, K % 32 == 0, 16-byte aligned
 * rows of input and weight and 8-byte aligned rows of output and bias; anything else returns
 * PMXHIP_UNSUPPORTED.  The kernels of this library are written for the decode step (M up to a few hundred rows:
 * bound by streaming the K * N * 2 weight bytes); they serve any M, 128 rows at a time, allocate nothing and add
 * their partial sums in a fixed order, so a call's result does not depend on timing.
 * workspace: at decode sizes there are fewer blocks of 64 output columns than CUs, so the k range is split over
 * several workgroups whose float32 partial tiles pass through `workspace` (the role of the reference's
 * cublas_workspace argument) and are added in a fixed order by a second kernel.
 * pmxhip_row_parallel_linear_workspace_size gives the bytes that serve (M, in_features, out_features) on the
 * current device (0 = none needed); with a NULL or smaller workspace the call still computes the same function,
 * one k range per column block (slower at decode sizes).  The workspace needs 16-byte alignment and no clearing.
 *
 * The _ex forms take flags.  PMXHIP_LINEAR_VENDOR_GEMM: from 384 rows on (a prefill chunk's query rows: a
 * compute-bound GEMM) the problem goes to hipBLASLt, as the reference's goes to cublasLt, if libhipblaslt.so can be
 * loaded (dlopen; there is no link-time dependency); where it cannot, or declines the problem, and below 384 rows,
 * this library's kernels run as without the flag.  That route is outside the rest of this header's contract: the
 * vendor library allocates on the host (its handle per device, descriptors per call), chooses its own summation
 * order, and is offered the caller's workspace (the _ex size query then asks for 64 MiB).  Its handle is created by
 * pmxhip_init_vendor_gemm() or by the first flagged call on a device, which must not come under stream capture. */
#define PMXHIP_LINEAR_VENDOR_GEMM 1
PMXHIP_API int64_t pmxhip_row_parallel_linear_workspace_size(int64_t m, int64_t in_features, int64_t out_features);
PMXHIP_API int pmxhip_row_parallel_linear(pmxhip_stream_t stream, const void* input, const void* weight, const void* bias,
                                          int64_t m, int64_t in_features, int64_t out_features, int64_t input_stride,
                                          int64_t weight_stride, int64_t output_stride, int64_t workspace_size,
                                          void* workspace, void* output);
PMXHIP_API int64_t pmxhip_row_parallel_linear_workspace_size_ex(int64_t m, int64_t in_features, int64_t out_features,
                                                                int32_t flags);
PMXHIP_API int pmxhip_row_parallel_linear_ex(pmxhip_stream_t stream, const void* input, const void* weight, const void* bias,
                                             int64_t m, int64_t in_features, int64_t out_features, int64_t input_stride,
                                             int64_t weight_stride, int64_t output_stride, int64_t workspace_size,
                                             void* workspace, void* output, int32_t flags);
/* Loads hipBLASLt and creates its handle on the current device (PMXHIP_LINEAR_VENDOR_GEMM); PMXHIP_UNSUPPORTED when
 * the library cannot be loaded.  Host only; allocates. */
PMXHIP_API int pmxhip_init_vendor_gemm(void);

/* One-time set-up on the current device, for callers that record their first step under stream capture: the
 * attribute calls of the kernels with large dynamic LDS (otherwise made at each kernel's first launch, which a
 * capturing stream refuses with PMXHIP_OTHER_ERROR) and the address of the static workspace.  Optional
 * otherwise; idempotent; host only.  No counterpart in the reference, whose cudaFuncSetAttribute calls sit in
 * its launch path (kernel.cu:1946). */
PMXHIP_API int pmxhip_init(void);

/* Library identity / build check (host only). */
PMXHIP_API const char* pmxhip_version(void);
PMXHIP_API const char* pmxhip_last_error(void); /* thread-local text of the last failure */

#ifdef __cplusplus
}
#endif
#endif /* PMX_HIP_C_API_H_ */
