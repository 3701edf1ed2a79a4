// The pmx operator class over the C ABI, the key_value_cache free function, and
// the C handle that lets a non-C++ host drive the class.
//
// heuristic_prepare keeps the reference's checks and derived values
// (src/ppl/kernel/llm/cuda/pmx/multi_head_cache_attention/utils.cu:68-131,
// 162-165, 210-214, 318-324) and replaces its launch heuristics (utils.cu:136-264)
// with the token-range plan of this implementation.
#include "pmx_hip/cache_attention.h"

#include <cmath>
#include <cstdio>
#include <cstring>
#include <new>

#include "pmx_hip/c_api.h"
#include "pmx_hip/key_value_cache.h"
#include "pmx_hip/kv_cache_reorder.h"
#include "pmx_hip/rotary_position_embedding.h"
#include "pmx_hip/row_parallel_linear.h"

namespace ppl { namespace kernel { namespace llm { namespace cuda { namespace pmx {

namespace {

constexpr int32_t UNIFORM_PAGE_SIZE = PMXHIP_PAGE_SIZE;

#define PMX_LOG_ERROR(...)                         \
    do {                                           \
        fprintf(stderr, "[pmx_hip] error: ");      \
        fprintf(stderr, __VA_ARGS__);              \
        fprintf(stderr, "\n");                     \
    } while (0)

ppl::common::RetCode to_retcode(int status)
{
    switch (status) {
        case PMXHIP_SUCCESS: return ppl::common::RC_SUCCESS;
        case PMXHIP_UNSUPPORTED: return ppl::common::RC_UNSUPPORTED;
        case PMXHIP_INVALID_VALUE: return ppl::common::RC_INVALID_VALUE;
        default: return ppl::common::RC_OTHER_ERROR;
    }
}

} // namespace

ppl::common::RetCode dynamic_batching_multi_head_cache_attention::heuristic_prepare(
    const hipDeviceProp_t& device_prop,
    const ppl::common::TensorShape* query_shape, const void* query,
    const ppl::common::TensorShape* current_key_shape, const void* current_key,
    const ppl::common::TensorShape* current_value_shape, const void* current_value,
    const ppl::common::TensorShape* attn_mask_shape, const void* attn_mask,
    const void* seqstarts, const void* kvstarts,
    const void* cachestarts, const void* start_pos,
    const void* alibi_slopes,
    const bool is_causal,
    const int64_t batch, const int64_t decoding_batches,
    const int64_t max_seqlen, const int64_t max_kvlen,
    const int64_t layer_idx, const int64_t num_layer,
    const int64_t num_heads, const int64_t num_kv_heads, const int64_t head_dim,
    const int32_t cache_mode, const int64_t page_size,
    const int64_t cache_stride_s, const int64_t cache_stride_l,
    const int64_t cache_stride_h, const int64_t cache_stride_kv,
    const int64_t cachestarts_stride_b,
    const bool enable_cache_prefill,
    const bool enable_sharemem_mhca, const bool enable_infinity_mhca, const bool enable_infinity_gqca,
    const int32_t specify_decoding_multi_block,
    const int32_t specify_decoding_tpb,
    void* cache, void* scale,
    const ppl::common::TensorShape* output_shape, void* output)
{
    // ---- shape checks, in the reference's order (utils.cu:68-95) ----
    if (query_shape->GetDim(1) != num_heads) {
        PMX_LOG_ERROR("currently do not support leading dim on query's num_heads");
        return ppl::common::RC_UNSUPPORTED;
    }
    if (output_shape->GetDim(1) != num_heads) {
        PMX_LOG_ERROR("currently do not support leading dim on output's num_heads");
        return ppl::common::RC_UNSUPPORTED;
    }
    if (current_key_shape->GetDim(1) != num_kv_heads) {
        PMX_LOG_ERROR("currently do not support leading dim on current_key's num_kv_heads");
        return ppl::common::RC_UNSUPPORTED;
    }
    if (current_value_shape->GetDim(1) != num_kv_heads) {
        PMX_LOG_ERROR("currently do not support leading dim on current_value's num_kv_heads");
        return ppl::common::RC_UNSUPPORTED;
    }
    if (cache_mode == 1 && page_size != UNIFORM_PAGE_SIZE) {
        PMX_LOG_ERROR("currently only support page_size == %d", UNIFORM_PAGE_SIZE);
        return ppl::common::RC_UNSUPPORTED;
    }

    constexpr int64_t VPT = 8;
    const int64_t num_kv_repeats = num_kv_heads > 0 ? num_heads / num_kv_heads : 0;
    if (num_kv_heads <= 0 || num_kv_heads * num_kv_repeats != num_heads) { // utils.cu:101-105
        PMX_LOG_ERROR("only support num_heads %% num_kv_heads == 0.");
        return ppl::common::RC_UNSUPPORTED;
    }

    // ---- derived values (utils.cu:107-131) ----
    const int64_t prefill_batches = batch - decoding_batches;
    // The prefill stage serves the head dims of the reference's flash attention (64, 96, 128, 256).  Others are
    // rejected here, not in forward_prefill, so that no stage is enqueued for a call that cannot complete.
    if (prefill_batches > 0 && max_seqlen > 0 && head_dim != 64 && head_dim != 96 && head_dim != 128 && head_dim != 256) {
        PMX_LOG_ERROR("prefill attention supports head dim 64, 96, 128 and 256, currently get %lld", (long long)head_dim);
        return ppl::common::RC_UNSUPPORTED;
    }
    const float attn_scale = float(1.0 / std::sqrt(float(head_dim)));
    const int64_t q_stride_s = query_shape->GetDim(1) * head_dim;
    const int64_t k_stride_s = current_key_shape->GetDim(1) * head_dim;
    const int64_t v_stride_s = current_value_shape->GetDim(1) * head_dim;
    const int64_t o_stride_s = output_shape->GetDim(1) * head_dim;

    int64_t mask_stride_s = 0, mask_stride_h = 0;
    if (attn_mask && attn_mask_shape && attn_mask_shape->CalcElementsExcludingPadding() > 0) {
        if (attn_mask_shape->GetDimCount() == 3) {
            mask_stride_h = attn_mask_shape->GetDim(1) * attn_mask_shape->GetDim(2);
            mask_stride_s = attn_mask_shape->GetDim(2);
        } else if (attn_mask_shape->GetDimCount() == 2) {
            mask_stride_s = attn_mask_shape->GetDim(1);
        } else {
            PMX_LOG_ERROR("attn_mask must be 2d or 3d");
            return ppl::common::RC_UNSUPPORTED;
        }
        if (mask_stride_s % VPT != 0) {
            PMX_LOG_ERROR("last dimension of attn_mask must be aligned with %lld", (long long)VPT);
            return ppl::common::RC_UNSUPPORTED;
        }
    }

    // ---- knob checks (utils.cu:162-165, 210-214) ----
    if (specify_decoding_multi_block < 0 || specify_decoding_multi_block > 2) {
        PMX_LOG_ERROR("specify_decoding_multi_block only accept 0/1/2");
        return ppl::common::RC_INVALID_VALUE;
    }
    int64_t decoding_threads_per_block = 256;
    if (specify_decoding_tpb) {
        if (specify_decoding_tpb != 256 && specify_decoding_tpb != 512) {
            PMX_LOG_ERROR("only support decoding tpb 256 or 512");
            return ppl::common::RC_INVALID_VALUE;
        }
        decoding_threads_per_block = specify_decoding_tpb; // recorded; the kernels here always run 256 threads
    }

    // ---- algorithm selection as the reference reports it (utils.cu:193-203, 244-264, 318-331).
    // Exactly one of the three must come out enabled; which one does not change the kernel here.
    const bool use_infinity_gqca = enable_infinity_gqca && decoding_batches > 0 &&
        (num_kv_repeats == 4 || num_kv_repeats == 6 || num_kv_repeats == 8 || num_kv_repeats == 16);
    bool use_sharemem_mhca = enable_sharemem_mhca && !use_infinity_gqca;
    bool use_infinity_mhca = false;
    if (enable_infinity_mhca && !use_infinity_gqca && decoding_batches > 0 && !use_sharemem_mhca) use_infinity_mhca = true;
    if ((use_infinity_gqca ? 1 : 0) + (use_infinity_mhca ? 1 : 0) + (use_sharemem_mhca ? 1 : 0) != 1) {
        PMX_LOG_ERROR("No algo to be used or more than one algo is selected, sharemem_mhca=%d, infinity_mhca=%d, infinity_gqca=%d",
                      (int)use_sharemem_mhca, (int)use_infinity_mhca, (int)use_infinity_gqca);
        return ppl::common::RC_OTHER_ERROR;
    }

    // ---- split plan of this implementation ----
    pmxhip_decode_plan plan;
    memset(&plan, 0, sizeof(plan));
    if (decoding_batches > 0) {
        const int32_t hint = specify_decoding_multi_block == 0 ? 1 : 0;
        const int rc = pmxhip_decode_plan_make(decoding_batches, num_heads, num_kv_heads, head_dim, max_kvlen,
                                               device_prop.multiProcessorCount, hint, &plan);
        // an unsupported head_dim is reported by forward_decode, as in the reference (kernel.cu:1975-2006)
        if (rc != PMXHIP_SUCCESS) memset(&plan, 0, sizeof(plan));
    }

    cfg.device_prop = const_cast<hipDeviceProp_t*>(&device_prop);
    cfg.datatype = query_shape->GetDataType();
    cfg.query = const_cast<void*>(query);
    cfg.current_key = const_cast<void*>(current_key);
    cfg.current_value = const_cast<void*>(current_value);
    cfg.attn_mask = const_cast<void*>(attn_mask);
    cfg.seqstarts = const_cast<void*>(seqstarts);
    cfg.kvstarts = const_cast<void*>(kvstarts);
    cfg.cachestarts = const_cast<void*>(cachestarts);
    cfg.start_pos = const_cast<void*>(start_pos);
    cfg.alibi_slopes = const_cast<void*>(alibi_slopes);
    cfg.cache = cache;
    cfg.scale = scale;
    cfg.output = output;
    cfg.is_causal = is_causal;
    cfg.batch = batch;
    cfg.decoding_batches = decoding_batches;
    cfg.max_seqlen = max_seqlen;
    cfg.max_kvlen = max_kvlen;
    cfg.prefill_query_rows = query_shape->GetDim(0) - decoding_batches; // decode sequences have one row each
    cfg.layer_idx = layer_idx;
    cfg.num_layer = num_layer;
    cfg.num_heads = num_heads;
    cfg.num_kv_heads = num_kv_heads;
    cfg.head_dim = head_dim;
    cfg.cache_mode = cache_mode;
    cfg.page_size = (int32_t)page_size;
    cfg.cache_stride_s = cache_stride_s;
    cfg.cache_stride_l = cache_stride_l;
    cfg.cache_stride_h = cache_stride_h;
    cfg.cache_stride_kv = cache_stride_kv;
    cfg.cachestarts_stride_b = cachestarts_stride_b;

    cfg.prefill_batches = prefill_batches;
    cfg.q_stride_s = q_stride_s;
    cfg.k_stride_s = k_stride_s;
    cfg.v_stride_s = v_stride_s;
    cfg.o_stride_s = o_stride_s;
    cfg.mask_stride_s = mask_stride_s;
    cfg.mask_stride_h = mask_stride_h;
    cfg.attn_scale = attn_scale;
    cfg.num_kv_repeats = num_kv_repeats;
    cfg.decoding_algo = use_infinity_gqca ? decoding_algo::INFINITY_GQCA
                                          : (use_infinity_mhca ? decoding_algo::INFINITY_MHCA : decoding_algo::SHAREMEM_MHCA);
    cfg.decoding_threads_per_block = decoding_threads_per_block;
    cfg.decoding_multi_block_size = plan.num_token_ranges > 0 ? plan.num_token_ranges : 1;
    cfg.decoding_multi_block_partial_out_size = plan.partial_out_size;
    cfg.decoding_multi_block_partial_log_sum_exp_size = plan.partial_ml_size;
    cfg.decoding_multi_block_counter_size = 0;
    cfg.workspace_size = plan.workspace_size;
    // short prefill chunks run on the decode step's kernel and keep their split-KV pieces in the same workspace (the
    // two stages follow each other on the stream)
    if (enable_cache_prefill && prefill_batches > 0 && !attn_mask && !alibi_slopes) {
        const int64_t chunk_ws = pmxhip_prefill_workspace_size(batch, decoding_batches, max_seqlen, max_kvlen, num_heads,
                                                               num_kv_heads, head_dim, device_prop.multiProcessorCount);
        if (chunk_ws > cfg.workspace_size) cfg.workspace_size = chunk_ws;
    }
    cfg.enable_cache_prefill = enable_cache_prefill;
    return ppl::common::RC_SUCCESS;
}

ppl::common::RetCode dynamic_batching_multi_head_cache_attention::forward_kvstore(const hipStream_t stream)
{
    pmxhip_kvstore_params p;
    memset(&p, 0, sizeof(p));
    p.current_key = cfg.current_key;
    p.current_value = cfg.current_value;
    p.seqstarts = static_cast<const int64_t*>(cfg.seqstarts);
    p.cachestarts = static_cast<const int64_t*>(cfg.cachestarts);
    p.start_pos = static_cast<const int64_t*>(cfg.start_pos);
    p.num_layer = cfg.num_layer;
    p.layer_idx = cfg.layer_idx;
    p.num_kv_heads = cfg.num_kv_heads;
    p.head_dim = cfg.head_dim;
    p.page_size = cfg.page_size;
    p.current_key_stride_s = cfg.k_stride_s;
    p.current_value_stride_s = cfg.v_stride_s;
    p.cache_stride_s = cfg.cache_stride_s;
    p.cache_stride_l = cfg.cache_stride_l;
    p.cache_stride_h = cfg.cache_stride_h;
    p.cache_stride_kv = cfg.cache_stride_kv;
    p.cachestarts_stride_b = cfg.cachestarts_stride_b;
    p.cache = cfg.cache;
    p.scale = cfg.scale;
    p.batch = cfg.batch;
    p.max_seqlen = cfg.max_seqlen;
    p.cache_mode = cfg.cache_mode;
    return to_retcode(pmxhip_kv_cache_quantize(&p, stream));
}

ppl::common::RetCode dynamic_batching_multi_head_cache_attention::forward_decode(const hipStream_t stream)
{
    if (cfg.decoding_batches <= 0) return ppl::common::RC_SUCCESS;
    pmxhip_decode_params p;
    memset(&p, 0, sizeof(p));
    p.query = cfg.query;
    p.attn_mask = cfg.attn_mask;
    p.output = cfg.output;
    p.cache = cfg.cache;
    p.scale = cfg.scale;
    p.cachestarts = static_cast<const int64_t*>(cfg.cachestarts);
    p.kvstarts = static_cast<const int64_t*>(cfg.kvstarts);
    p.attn_scale = cfg.attn_scale;
    p.layer_idx = cfg.layer_idx;
    p.num_kv_repeats = cfg.num_kv_repeats;
    p.page_size = cfg.page_size;
    p.query_stride_s = cfg.q_stride_s;
    p.output_stride_s = cfg.o_stride_s;
    p.mask_stride_s = cfg.mask_stride_s;
    p.mask_stride_h = cfg.mask_stride_h;
    p.cache_stride_s = cfg.cache_stride_s;
    p.cache_stride_l = cfg.cache_stride_l;
    p.cache_stride_h = cfg.cache_stride_h;
    p.cache_stride_kv = cfg.cache_stride_kv;
    p.cachestarts_stride_b = cfg.cachestarts_stride_b;
    p.decoding_batches = cfg.decoding_batches;
    p.num_heads = cfg.num_heads;
    p.num_kv_heads = cfg.num_kv_heads;
    p.head_dim = cfg.head_dim;
    p.cache_mode = cfg.cache_mode;
    p.num_token_ranges = (int32_t)cfg.decoding_multi_block_size;
    p.workspace = cfg.workspace;
    p.workspace_size = cfg.workspace_size;
    const int rc = pmxhip_decode_attention(&p, stream);
    if (rc != PMXHIP_SUCCESS) {
        // the reference folds every decode dispatch failure into RC_UNSUPPORTED (kernel.cu:2118-2121); what is not a
        // matter of the configuration keeps its own code (a bad argument, a first launch under stream capture)
        PMX_LOG_ERROR("decode stage rejected the configuration");
        return rc == PMXHIP_UNSUPPORTED ? ppl::common::RC_UNSUPPORTED : to_retcode(rc);
    }
    return ppl::common::RC_SUCCESS;
}

ppl::common::RetCode dynamic_batching_multi_head_cache_attention::forward_prefill(const hipStream_t stream)
{
    if (cfg.prefill_batches <= 0) return ppl::common::RC_SUCCESS;
    if (cfg.datatype != ppl::common::DATATYPE_FLOAT16) { // flash_attn2/fmha.cu:75
        PMX_LOG_ERROR("prefill attention only supports fp16");
        return ppl::common::RC_UNSUPPORTED;
    }
    pmxhip_prefill_params p;
    memset(&p, 0, sizeof(p));
    p.query = cfg.query;
    p.output = cfg.output;
    p.cache = cfg.cache;
    p.scale = cfg.scale;
    p.seqstarts = static_cast<const int64_t*>(cfg.seqstarts);
    p.kvstarts = static_cast<const int64_t*>(cfg.kvstarts);
    p.cachestarts = static_cast<const int64_t*>(cfg.cachestarts);
    p.attn_scale = cfg.attn_scale;
    p.is_causal = cfg.is_causal ? 1 : 0;
    p.batch = cfg.batch;
    p.decoding_batches = cfg.decoding_batches;
    p.max_seqlen = cfg.max_seqlen;
    p.max_kvlen = cfg.max_kvlen;
    p.layer_idx = cfg.layer_idx;
    p.num_heads = cfg.num_heads;
    p.num_kv_heads = cfg.num_kv_heads;
    p.head_dim = cfg.head_dim;
    p.cache_mode = cfg.cache_mode;
    p.page_size = cfg.page_size;
    p.query_stride_s = cfg.q_stride_s;
    p.output_stride_s = cfg.o_stride_s;
    p.cache_stride_s = cfg.cache_stride_s;
    p.cache_stride_l = cfg.cache_stride_l;
    p.cache_stride_h = cfg.cache_stride_h;
    p.cache_stride_kv = cfg.cache_stride_kv;
    p.cachestarts_stride_b = cfg.cachestarts_stride_b;
    p.attn_mask = cfg.attn_mask;
    p.mask_stride_s = cfg.mask_stride_s;
    p.mask_stride_h = cfg.mask_stride_h;
    p.alibi_slopes = static_cast<const float*>(cfg.alibi_slopes);
    p.prefill_query_rows = cfg.prefill_query_rows;
    p.workspace = cfg.workspace;
    p.workspace_size = cfg.workspace_size;
    if (!cfg.enable_cache_prefill) { // kernel.cu:2181-2212: the step's own fp16 K/V only, no cache read
        p.current_key = cfg.current_key;
        p.current_value = cfg.current_value;
        p.key_stride_s = cfg.k_stride_s;
        p.value_stride_s = cfg.v_stride_s;
    }
    return to_retcode(pmxhip_prefill_attention(&p, stream));
}

ppl::common::RetCode dynamic_batching_multi_head_cache_attention::forward(const hipStream_t stream)
{
    // First failure wins (the reference keeps only the last stage's status, kernel.cu:2219-2240).
    ppl::common::RetCode ret = forward_kvstore(stream);
    if (ret != ppl::common::RC_SUCCESS) {
        PMX_LOG_ERROR("kv_store stage failed.");
        return ret;
    }
    ret = forward_decode(stream);
    if (ret != ppl::common::RC_SUCCESS) {
        PMX_LOG_ERROR("decode stage failed.");
        return ret;
    }
    ret = forward_prefill(stream);
    if (ret != ppl::common::RC_SUCCESS) PMX_LOG_ERROR("prefill stage failed.");
    return ret;
}

ppl::common::RetCode dynamic_batching_multi_head_cache_attention::forward(const hipStream_t stream, const hipStream_t side_stream,
                                                                          const hipEvent_t fork_event, const hipEvent_t join_event)
{
    // the prefill stage on the short-chunk route writes its pieces into the workspace that the decode stage is using
    const bool shared_workspace =
        cfg.workspace != nullptr && cfg.decoding_multi_block_size > 1 && cfg.enable_cache_prefill && !cfg.attn_mask && !cfg.alibi_slopes &&
        pmxhip_prefill_workspace_size(cfg.batch, cfg.decoding_batches, cfg.max_seqlen, cfg.max_kvlen, cfg.num_heads, cfg.num_kv_heads,
                                      cfg.head_dim, cfg.device_prop ? cfg.device_prop->multiProcessorCount : 0) > 0;
    if (cfg.decoding_batches <= 0 || cfg.prefill_batches <= 0 || side_stream == stream || shared_workspace) return forward(stream);
    if (!fork_event || !join_event) {
        PMX_LOG_ERROR("forward on two streams needs a fork and a join event");
        return ppl::common::RC_INVALID_VALUE;
    }
    ppl::common::RetCode ret = forward_kvstore(stream);
    if (ret != ppl::common::RC_SUCCESS) {
        PMX_LOG_ERROR("kv_store stage failed.");
        return ret;
    }
    if (hipEventRecord(fork_event, stream) != hipSuccess || hipStreamWaitEvent(side_stream, fork_event, 0) != hipSuccess) {
        PMX_LOG_ERROR("forward on two streams: the fork failed: %s", hipGetErrorString(hipGetLastError()));
        return ppl::common::RC_OTHER_ERROR;
    }
    // from here the side stream is part of the step (and of a capture): it is joined whatever the stages return
    const ppl::common::RetCode ret_decode = forward_decode(side_stream);
    const bool joined_side = hipEventRecord(join_event, side_stream) == hipSuccess;
    const ppl::common::RetCode ret_prefill = forward_prefill(stream);
    if (!joined_side || hipStreamWaitEvent(stream, join_event, 0) != hipSuccess) {
        PMX_LOG_ERROR("forward on two streams: the join failed: %s", hipGetErrorString(hipGetLastError()));
        return ppl::common::RC_OTHER_ERROR;
    }
    if (ret_decode != ppl::common::RC_SUCCESS) {
        PMX_LOG_ERROR("decode stage failed.");
        return ret_decode;
    }
    if (ret_prefill != ppl::common::RC_SUCCESS) PMX_LOG_ERROR("prefill stage failed.");
    return ret_prefill;
}

ppl::common::RetCode dynamic_batching_key_value_cache(
    const hipStream_t stream,
    const ppl::common::TensorShape* current_key_shape, const void* current_key,
    const ppl::common::TensorShape* current_value_shape, const void* current_value,
    const void* seqstarts, const void* cachestarts, const void* start_pos,
    const int64_t batch, const int64_t max_seqlen,
    const int64_t num_layer, const int64_t layer_idx,
    const int64_t num_kv_heads, const int64_t head_dim,
    const int32_t cache_mode, const int64_t page_size,
    const int64_t cache_stride_s, const int64_t cache_stride_l,
    const int64_t cache_stride_h, const int64_t cache_stride_kv,
    const int64_t cachestarts_stride_b,
    void* cache, void* scale)
{
    if (current_key_shape->GetDim(1) != num_kv_heads || current_value_shape->GetDim(1) != num_kv_heads) {
        PMX_LOG_ERROR("currently do not support leading dim on current_key/value's num_kv_heads");
        return ppl::common::RC_UNSUPPORTED;
    }
    return to_retcode(pmxhip_key_value_cache(
        stream, current_key, current_value, static_cast<const int64_t*>(seqstarts),
        static_cast<const int64_t*>(cachestarts), static_cast<const int64_t*>(start_pos), batch, max_seqlen, num_layer,
        layer_idx, num_kv_heads, head_dim, cache_mode, page_size, cache_stride_s, cache_stride_l, cache_stride_h,
        cache_stride_kv, cachestarts_stride_b, cache, scale));
}

static pmxhip_reorder_stride to_c_stride(const Stride& s)
{
    pmxhip_reorder_stride r;
    r.p_stride_cache = s.p_stride_cache; r.l_stride_cache = s.l_stride_cache; r.kv_stride_cache = s.kv_stride_cache;
    r.h_stride_cache = s.h_stride_cache; r.t_stride_cache = s.t_stride_cache; r.d_stride_cache = s.d_stride_cache;
    r.p_stride_scale = s.p_stride_scale; r.l_stride_scale = s.l_stride_scale; r.kv_stride_scale = s.kv_stride_scale;
    r.h_stride_scale = s.h_stride_scale; r.t_stride_scale = s.t_stride_scale; r.d_stride_scale = s.d_stride_scale;
    return r;
}

ppl::common::RetCode kv_cache_reorder(
    hipStream_t stream, const void* kv_cache, const void* kv_scale, const void* page_ids,
    const Stride& src_stride, const Stride& dst_stride,
    int64_t page_nums, int64_t layers, int64_t kv_heads, int64_t tokens, int64_t head_dim, int64_t group_size,
    int64_t tp_rank, int64_t tp_size, void* outer_mem)
{
    const pmxhip_reorder_stride s = to_c_stride(src_stride), d = to_c_stride(dst_stride);
    return to_retcode(pmxhip_kv_cache_reorder(stream, kv_cache, kv_scale, static_cast<const int64_t*>(page_ids), &s, &d, page_nums,
                                              layers, kv_heads, tokens, head_dim, group_size, tp_rank, tp_size, outer_mem));
}

ppl::common::RetCode kv_cache_invert_reorder(
    hipStream_t stream, const void* outer_mem, const void* page_ids,
    const Stride& src_stride, const Stride& dst_stride,
    int64_t page_nums, int64_t layers, int64_t kv_heads, int64_t tokens, int64_t head_dim, int64_t group_size,
    int64_t tp_rank, int64_t tp_size, void* kv_cache, void* kv_scale)
{
    const pmxhip_reorder_stride s = to_c_stride(src_stride), d = to_c_stride(dst_stride);
    return to_retcode(pmxhip_kv_cache_invert_reorder(stream, outer_mem, static_cast<const int64_t*>(page_ids), &s, &d, page_nums,
                                                     layers, kv_heads, tokens, head_dim, group_size, tp_rank, tp_size, kv_cache,
                                                     kv_scale));
}

static ppl::common::RetCode fill_rope_params(
    pmxhip_rope_params& p,
    const ppl::common::TensorShape* query_shape, const void* query, const ppl::common::TensorShape* key_shape, const void* key,
    const void* start_pos, const void* seqstarts, const float theta, const int32_t bypass_key, const int64_t rotary_dim,
    const int64_t batch, const int64_t num_heads, const int64_t num_key_heads, const int64_t max_seqlen,
    const int64_t max_position_embeddings, const rope_scaling_t scaling_type, const float scaling_factor,
    const ppl::common::TensorShape* rotated_query_shape, void* rotated_query,
    const ppl::common::TensorShape* rotated_key_shape, void* rotated_key)
{
    // checks of rotary_position_embedding.cu:368-398
    if (query_shape->GetDataType() != ppl::common::DATATYPE_FLOAT16) {
        PMX_LOG_ERROR("only support fp16");
        return ppl::common::RC_UNSUPPORTED;
    }
    if (query_shape->GetDimCount() != 3 || key_shape->GetDimCount() != 3 || rotated_query_shape->GetDimCount() != 3 ||
        (rotated_key && rotated_key_shape->GetDimCount() != 3)) {
        PMX_LOG_ERROR("query, key, rotated_query and rotated_key must have 3 dims");
        return ppl::common::RC_INVALID_VALUE;
    }
    const int64_t head_dim = query_shape->GetDim(2);
    if (head_dim % 2 != 0 || rotary_dim % 2 != 0) {
        PMX_LOG_ERROR("head_dim and rotary_dim should be even numbers");
        return ppl::common::RC_INVALID_VALUE;
    }
    memset(&p, 0, sizeof(p));
    p.query = query;
    p.key = key;
    p.start_pos = static_cast<const int64_t*>(start_pos);
    p.seqstarts = static_cast<const int64_t*>(seqstarts);
    p.theta = theta;
    p.bypass_key = bypass_key;
    p.rotary_dim = rotary_dim;
    p.batch = batch;
    p.num_heads = num_heads;
    p.num_key_heads = num_key_heads;
    p.head_dim = head_dim;
    p.max_seqlen = max_seqlen;
    p.max_position_embeddings = max_position_embeddings;
    p.scaling_type = scaling_type;
    p.scaling_factor = scaling_factor;
    p.query_stride_s = query_shape->GetDim(1) * head_dim; // lines 411-414: dim[1] is the leading dim of heads
    p.key_stride_s = key_shape->GetDim(1) * head_dim;
    p.rotated_query_stride_s = rotated_query_shape->GetDim(1) * head_dim;
    p.rotated_key_stride_s = rotated_key ? rotated_key_shape->GetDim(1) * head_dim : 0;
    p.rotated_query = rotated_query;
    p.rotated_key = rotated_key;
    return ppl::common::RC_SUCCESS;
}

ppl::common::RetCode dynamic_batching_rotary_position_embedding(
    hipStream_t stream,
    const ppl::common::TensorShape* query_shape, const void* query,
    const ppl::common::TensorShape* key_shape, const void* key,
    const void* start_pos, const void* seqstarts,
    const float theta, const int32_t bypass_key, const int64_t rotary_dim,
    const int64_t batch, const int64_t num_heads, const int64_t num_key_heads,
    const int64_t max_seqlen, const int64_t max_position_embeddings,
    const rope_scaling_t scaling_type, const float scaling_factor,
    const ppl::common::TensorShape* rotated_query_shape, void* rotated_query,
    const ppl::common::TensorShape* rotated_key_shape, void* rotated_key)
{
    pmxhip_rope_params p;
    const ppl::common::RetCode rc = fill_rope_params(p, query_shape, query, key_shape, key, start_pos, seqstarts, theta, bypass_key,
                                                     rotary_dim, batch, num_heads, num_key_heads, max_seqlen,
                                                     max_position_embeddings, scaling_type, scaling_factor, rotated_query_shape,
                                                     rotated_query, rotated_key_shape, rotated_key);
    if (rc != ppl::common::RC_SUCCESS) return rc;
    return to_retcode(pmxhip_rotary_position_embedding(&p, stream));
}

ppl::common::RetCode dynamic_batching_rotary_position_embedding_kv_cache(
    hipStream_t stream,
    const ppl::common::TensorShape* query_shape, const void* query,
    const ppl::common::TensorShape* key_shape, const void* key,
    const ppl::common::TensorShape* value_shape, const void* current_value,
    const void* start_pos, const void* seqstarts,
    const float theta, const int32_t bypass_key, const int64_t rotary_dim,
    const int64_t batch, const int64_t num_heads, const int64_t num_key_heads,
    const int64_t max_seqlen, const int64_t max_position_embeddings,
    const rope_scaling_t scaling_type, const float scaling_factor,
    const ppl::common::TensorShape* rotated_query_shape, void* rotated_query,
    const ppl::common::TensorShape* rotated_key_shape, void* rotated_key,
    const void* cachestarts, const int64_t num_layer, const int64_t layer_idx,
    const int32_t cache_mode, const int64_t page_size,
    const int64_t cache_stride_s, const int64_t cache_stride_l, const int64_t cache_stride_h,
    const int64_t cache_stride_kv, const int64_t cachestarts_stride_b,
    void* cache, void* scale)
{
    pmxhip_rope_params p;
    const ppl::common::RetCode rc = fill_rope_params(p, query_shape, query, key_shape, key, start_pos, seqstarts, theta, bypass_key,
                                                     rotary_dim, batch, num_heads, num_key_heads, max_seqlen,
                                                     max_position_embeddings, scaling_type, scaling_factor, rotated_query_shape,
                                                     rotated_query, rotated_key_shape, rotated_key);
    if (rc != ppl::common::RC_SUCCESS) return rc;
    if (value_shape->GetDimCount() != 3) {
        PMX_LOG_ERROR("current_value's dim should be 3");
        return ppl::common::RC_INVALID_VALUE;
    }
    pmxhip_kvstore_params st;
    memset(&st, 0, sizeof(st));
    st.current_key = key;
    st.current_value = current_value;
    st.seqstarts = p.seqstarts;
    st.cachestarts = static_cast<const int64_t*>(cachestarts);
    st.start_pos = p.start_pos;
    st.num_layer = num_layer;
    st.layer_idx = layer_idx;
    st.num_kv_heads = num_key_heads;
    st.head_dim = p.head_dim;
    st.page_size = (int32_t)page_size;
    st.current_key_stride_s = p.key_stride_s;
    st.current_value_stride_s = value_shape->GetDim(1) * p.head_dim;
    st.cache_stride_s = cache_stride_s;
    st.cache_stride_l = cache_stride_l;
    st.cache_stride_h = cache_stride_h;
    st.cache_stride_kv = cache_stride_kv;
    st.cachestarts_stride_b = cachestarts_stride_b;
    st.cache = cache;
    st.scale = scale;
    st.batch = batch;
    st.max_seqlen = max_seqlen;
    st.cache_mode = cache_mode;
    return to_retcode(pmxhip_rope_kv_cache_quantize(&p, &st, stream));
}

ppl::common::RetCode row_parallel_linear(
    const hipStream_t stream,
    const ppl::common::TensorShape* input_shape, const void* input,
    const ppl::common::TensorShape* weight_shape, const void* weight,
    const ppl::common::TensorShape* bias_shape, const void* bias,
    const int64_t in_features, const int64_t out_features,
    const bool input_is_parallel,
    const int64_t workspace_size, void* workspace,
    const ppl::common::TensorShape* output_shape, void* output,
    const bool use_vendor_gemm)
{
    (void)bias_shape;
    (void)output_shape;
    if (!input_is_parallel) { // row_parallel_linear.cu:46-49
        PMX_LOG_ERROR("currnetly only support parallel input");
        return ppl::common::RC_UNSUPPORTED;
    }
    if (!input_shape || !weight_shape) {
        PMX_LOG_ERROR("row_parallel_linear: null shape");
        return ppl::common::RC_INVALID_VALUE;
    }
    if (input_shape->GetDataType() != ppl::common::DATATYPE_FLOAT16 || weight_shape->GetDataType() != ppl::common::DATATYPE_FLOAT16) {
        PMX_LOG_ERROR("row_parallel_linear only supports fp16");
        return ppl::common::RC_UNSUPPORTED;
    }
    // M = all dimensions of the input but the last (row_parallel_linear.cu:55)
    int64_t m = 1;
    for (uint32_t i = 0; i + 1 < input_shape->GetDimCount(); ++i) m *= input_shape->GetDim(i);
    return to_retcode(pmxhip_row_parallel_linear_ex(stream, input, weight, bias, m, in_features, out_features, in_features, in_features,
                                                    out_features, workspace_size, workspace, output,
                                                    use_vendor_gemm ? PMXHIP_LINEAR_VENDOR_GEMM : 0));
}

ppl::common::RetCode row_parallel_linear(
    const hipStream_t stream,
    const cublasLtHandle_t& cublaslt_handle, const cublasLtMatmulAlgo_t* algo,
    const ppl::common::TensorShape* input_shape, const void* input,
    const ppl::common::TensorShape* weight_shape, const void* weight,
    const ppl::common::TensorShape* bias_shape, const void* bias,
    const int64_t in_features, const int64_t out_features,
    const ppl::common::NcclParam* nccl_param, const bool input_is_parallel, void* split_buffer,
    const int64_t cublas_workspace_size, void* cublas_workspace,
    const ppl::common::TensorShape* output_shape, void* output,
    const bool use_vendor_gemm)
{
    (void)cublaslt_handle; // the GEMM runs on this library's kernels (or on a hipBLASLt handle of its own)
    (void)algo;
    (void)split_buffer;    // the reference's scratch for input_is_parallel = false, which it rejects as well
    if (nccl_param && nccl_param->size > 1) { // row_parallel_linear.cu:83-97: the all-reduce over the ranks
        PMX_LOG_ERROR("row_parallel_linear: a communicator of %d ranks; this build runs on one GPU and has no all-reduce",
                      nccl_param->size);
        return ppl::common::RC_UNSUPPORTED;
    }
    return row_parallel_linear(stream, input_shape, input, weight_shape, weight, bias_shape, bias, in_features, out_features,
                               input_is_parallel, cublas_workspace_size, cublas_workspace, output_shape, output, use_vendor_gemm);
}

int64_t row_parallel_linear_workspace_size(const int64_t m, const int64_t in_features, const int64_t out_features,
                                           const bool use_vendor_gemm)
{
    return pmxhip_row_parallel_linear_workspace_size_ex(m, in_features, out_features, use_vendor_gemm ? PMXHIP_LINEAR_VENDOR_GEMM : 0);
}

}}}}} // namespace ppl::kernel::llm::cuda::pmx

// ---- C handle over the class ---------------------------------------------------

using mhca_class = ppl::kernel::llm::cuda::pmx::dynamic_batching_multi_head_cache_attention;

struct pmxhip_mhca {
    mhca_class op;
    hipDeviceProp_t prop; // heuristic_prepare keeps a pointer to it
    bool prepared;
};

namespace {

ppl::common::TensorShape to_shape(const pmxhip_tensor_shape& s)
{
    ppl::common::TensorShape t;
    t.SetDataType((ppl::common::datatype_t)s.data_type);
    const int n = s.dim_count < 0 ? 0 : (s.dim_count > 4 ? 4 : s.dim_count);
    t.SetDimCount((uint32_t)n);
    for (int i = 0; i < n; ++i) t.SetDim((uint32_t)i, s.dims[i]);
    return t;
}

} // namespace

extern "C" {

pmxhip_mhca_t pmxhip_mhca_create(void)
{
    pmxhip_mhca* h = new (std::nothrow) pmxhip_mhca();
    if (h) {
        memset(&h->prop, 0, sizeof(h->prop));
        h->prepared = false;
    }
    return h;
}

void pmxhip_mhca_destroy(pmxhip_mhca_t op) { delete op; }

int pmxhip_mhca_heuristic_prepare(pmxhip_mhca_t h, const pmxhip_mhca_prepare_args* a)
{
    if (!h || !a) return PMXHIP_INVALID_VALUE;
    h->prop.multiProcessorCount = a->compute_units;
    h->prop.sharedMemPerBlockOptin = (size_t)a->shared_mem_per_block_optin;
    const ppl::common::TensorShape qs = to_shape(a->query_shape), ks = to_shape(a->current_key_shape),
                                   vs = to_shape(a->current_value_shape), ms = to_shape(a->attn_mask_shape),
                                   os = to_shape(a->output_shape);
    const ppl::common::RetCode rc = h->op.heuristic_prepare(
        h->prop, &qs, a->query, &ks, a->current_key, &vs, a->current_value, &ms, a->attn_mask, a->seqstarts, a->kvstarts,
        a->cachestarts, a->start_pos, a->alibi_slopes, a->is_causal != 0, a->batch, a->decoding_batches, a->max_seqlen,
        a->max_kvlen, a->layer_idx, a->num_layer, a->num_heads, a->num_kv_heads, a->head_dim, a->cache_mode, a->page_size,
        a->cache_stride_s, a->cache_stride_l, a->cache_stride_h, a->cache_stride_kv, a->cachestarts_stride_b,
        a->enable_cache_prefill != 0, a->enable_sharemem_mhca != 0, a->enable_infinity_mhca != 0,
        a->enable_infinity_gqca != 0, a->specify_decoding_multi_block, a->specify_decoding_tpb, a->cache, a->scale, &os,
        a->output);
    h->prepared = rc == ppl::common::RC_SUCCESS;
    return (int)rc;
}

int pmxhip_mhca_get_derived(pmxhip_mhca_t h, pmxhip_mhca_derived* out)
{
    if (!h || !out || !h->prepared) return PMXHIP_INVALID_VALUE;
    const mhca_class::config& c = h->op.cfg;
    out->prefill_batches = c.prefill_batches;
    out->q_stride_s = c.q_stride_s;
    out->k_stride_s = c.k_stride_s;
    out->v_stride_s = c.v_stride_s;
    out->o_stride_s = c.o_stride_s;
    out->mask_stride_s = c.mask_stride_s;
    out->mask_stride_h = c.mask_stride_h;
    out->attn_scale = c.attn_scale;
    out->num_kv_repeats = c.num_kv_repeats;
    out->decoding_algo = c.decoding_algo;
    out->decoding_threads_per_block = c.decoding_threads_per_block;
    out->decoding_multi_block_size = c.decoding_multi_block_size;
    out->decoding_multi_block_partial_out_size = c.decoding_multi_block_partial_out_size;
    out->decoding_multi_block_partial_log_sum_exp_size = c.decoding_multi_block_partial_log_sum_exp_size;
    out->decoding_multi_block_counter_size = c.decoding_multi_block_counter_size;
    out->workspace_size = c.workspace_size;
    return PMXHIP_SUCCESS;
}

int pmxhip_mhca_set_workspace(pmxhip_mhca_t h, void* workspace)
{
    if (!h || !h->prepared) return PMXHIP_INVALID_VALUE;
    h->op.cfg.workspace = workspace;
    return PMXHIP_SUCCESS;
}

int pmxhip_mhca_forward_kvstore(pmxhip_mhca_t h, pmxhip_stream_t stream)
{
    if (!h || !h->prepared) return PMXHIP_INVALID_VALUE;
    return (int)h->op.forward_kvstore(stream);
}

int pmxhip_mhca_forward_decode(pmxhip_mhca_t h, pmxhip_stream_t stream)
{
    if (!h || !h->prepared) return PMXHIP_INVALID_VALUE;
    return (int)h->op.forward_decode(stream);
}

int pmxhip_mhca_forward_prefill(pmxhip_mhca_t h, pmxhip_stream_t stream)
{
    if (!h || !h->prepared) return PMXHIP_INVALID_VALUE;
    return (int)h->op.forward_prefill(stream);
}

int pmxhip_mhca_forward(pmxhip_mhca_t h, pmxhip_stream_t stream)
{
    if (!h || !h->prepared) return PMXHIP_INVALID_VALUE;
    return (int)h->op.forward(stream);
}

int pmxhip_mhca_forward_streams(pmxhip_mhca_t h, pmxhip_stream_t stream, pmxhip_stream_t side_stream, void* fork_event,
                                void* join_event)
{
    if (!h || !h->prepared) return PMXHIP_INVALID_VALUE;
    return (int)h->op.forward(stream, side_stream, static_cast<hipEvent_t>(fork_event), static_cast<hipEvent_t>(join_event));
}

} // extern "C"
