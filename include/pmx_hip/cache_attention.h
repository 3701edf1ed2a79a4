/*
 * Operator interface of the int8-KV dynamic-batching cache attention on MI355X.
 *
 * Source-compatible with the reference operator declared at
 * include/ppl/kernel/llm/cuda/pmx/multi_head_cache_attention.h:25-159 -- same
 * namespace (the `cuda` component is kept on purpose), class name, cfg field
 * names, heuristic_prepare argument order (reference lines 107-148) and stage
 * functions (reference lines 152-158) -- with hipStream_t / hipDeviceProp_t in
 * place of the CUDA types.  A call site written for the reference compiles
 * against this header once its include line is switched.
 *
 * Behaviour that differs on purpose:
 *   * forward() reports the FIRST failing stage (the reference overwrites the
 *     status stage by stage and reports only the last, kernel.cu:2219-2240).
 *   * enable_sharemem_mhca / enable_infinity_mhca / enable_infinity_gqca /
 *     specify_decoding_tpb are checked as the reference checks them
 *     (utils.cu:162-165, 210-214, 318-324) but select nothing: one decode
 *     kernel family serves MHA and GQA.  cfg.decoding_algo reports the
 *     reference's name for the closest equivalent.
 *   * specify_decoding_multi_block 0 = a single kv-token range (no workspace),
 *     1 and 2 = as many ranges as fill the GPU.  cfg.decoding_multi_block_size
 *     holds the range count.
 *   * cfg.workspace_size follows this implementation (float32 partial outputs
 *     and (max, sum) pairs; no arrival counters), not utils.cu:334-343.
 *   * Decode and prefill serve head_dim 64, 96, 128 and 256 (the reference's set: kernel.cu:1962 and the
 *     flash_fwd_hdim{64,96,128,256}_int8_g8 kernels).  heuristic_prepare rejects a batch with prefill
 *     sequences at any other head_dim with RC_UNSUPPORTED, before anything is enqueued.
 */
#ifndef PMX_HIP_CACHE_ATTENTION_H_
#define PMX_HIP_CACHE_ATTENTION_H_

#include <hip/hip_runtime_api.h>

#include <cstdint>

#include "pmx_hip/ppl_common_compat.h"

namespace ppl { namespace kernel { namespace llm { namespace cuda { namespace pmx {

class PMXHIP_CXX_API dynamic_batching_multi_head_cache_attention {
public:
    typedef int32_t decoding_algo_t;
    struct decoding_algo {
        static const decoding_algo_t UNKNOWN = 0, SHAREMEM_MHCA = 1, INFINITY_MHCA = 2, INFINITY_GQCA = 3;
    };

    struct config {
        // -- copied in by heuristic_prepare --
        hipDeviceProp_t* device_prop; // points at the caller's struct; must outlive forward*()
        ppl::common::datatype_t datatype;
        void *query, *current_key, *current_value, *attn_mask;
        void *seqstarts, *kvstarts, *cachestarts, *start_pos, *alibi_slopes;
        void *cache, *scale;
        void* output;
        bool is_causal;
        int64_t batch, decoding_batches, max_seqlen, max_kvlen;
        int64_t layer_idx, num_layer, num_heads, num_kv_heads, head_dim;
        int32_t cache_mode, page_size;
        int32_t page_shift, page_mask; // present in the reference's struct, never set there either
        int64_t cache_stride_s, cache_stride_l, cache_stride_h, cache_stride_kv, cachestarts_stride_b;
        // -- derived by heuristic_prepare --
        int64_t prefill_batches;
        int64_t q_stride_s, k_stride_s, v_stride_s, o_stride_s;
        int64_t mask_stride_s, mask_stride_h;
        float attn_scale;
        int64_t num_kv_repeats;
        decoding_algo_t decoding_algo;
        int64_t decoding_threads_per_block;
        int64_t decoding_multi_block_size;
        int64_t decoding_multi_block_partial_out_size;
        int64_t decoding_multi_block_partial_log_sum_exp_size;
        int64_t decoding_multi_block_counter_size; // always 0 here
        int64_t workspace_size;
        void* workspace; // the caller assigns this after heuristic_prepare, before forward*()
        bool enable_cache_prefill;
        int64_t prefill_query_rows; // not in the reference: rows of query beyond the decode rows.  A hint that lets the
                                    // prefill stage launch fewer workgroups; 0 = unknown.  A wrong value costs time only:
                                    // the stage's workgroups walk every query tile of the batch whatever the launch size.
    } cfg{};

    // Validates, derives strides / attn_scale / split plan and fills cfg.  Host only.
    ppl::common::RetCode heuristic_prepare(
        const hipDeviceProp_t& device_prop,
        const ppl::common::TensorShape* query_shape, const void* query,                 // (Sq, Hq, D)
        const ppl::common::TensorShape* current_key_shape, const void* current_key,     // (Skv, KVH, D)
        const ppl::common::TensorShape* current_value_shape, const void* current_value, // (Skv, KVH, D)
        const ppl::common::TensorShape* attn_mask_shape, const void* attn_mask, // (Sq, align8(Skv)) or (Hq, Sq, align8(Skv))
        const void* seqstarts, const void* kvstarts, // int64 (B + 1) each
        const void* cachestarts, const void* start_pos, // int64 (B) or (B, MaxP); int64 (B)
        const void* alibi_slopes, // float32 (Hq) or null; applied by the prefill stage only, as in the reference
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
        const int32_t specify_decoding_multi_block, // 0, 1 or 2
        const int32_t specify_decoding_tpb,         // 0, 256 or 512
        void* cache, void* scale, // int8 cache and float16 group-of-8 scales, same strides (/8)
        const ppl::common::TensorShape* output_shape, void* output); // (Sq, Hq, D)

    // Stages, all asynchronous on `stream`; kvstore first.
    ppl::common::RetCode forward_kvstore(const hipStream_t stream);
    ppl::common::RetCode forward_decode(const hipStream_t stream);
    ppl::common::RetCode forward_prefill(const hipStream_t stream);
    ppl::common::RetCode forward(const hipStream_t stream);
    // forward() of a mixed step with its two attention stages side by side (no counterpart in the reference, whose
    // forward runs the three stages in one stream order, kernel.cu:2219-2240): once the new rows are in the cache
    // the decode stage and the prefill stage touch disjoint sequences and output rows, so the decode stage goes to
    // `side_stream` -- forked from `stream` behind the append with `fork_event`, joined back into `stream` with
    // `join_event` -- and its workgroups fill the compute units that the prefill kernel's tail leaves idle.  Streams
    // and events are the caller's (both streams of the default priority; the events may be created without
    // timing); the library creates nothing, so the call can be recorded into a HIP graph from `stream`.  When the
    // call returns, everything it enqueued is ordered before later work on `stream`.  A step that is not mixed, a
    // side stream equal to `stream`, and a step whose prefill stage shares the workspace with the decode stage
    // (short chunks on the decode kernels) run exactly like forward(stream).
    ppl::common::RetCode forward(const hipStream_t stream, const hipStream_t side_stream, const hipEvent_t fork_event,
                                 const hipEvent_t join_event);
};

}}}}} // namespace ppl::kernel::llm::cuda::pmx

#endif // PMX_HIP_CACHE_ATTENTION_H_
