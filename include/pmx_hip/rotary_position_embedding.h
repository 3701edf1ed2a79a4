/*
 * Rotary position embedding for dynamic batches on MI355X, and its fusion with the int8 KV append.
 *
 * dynamic_batching_rotary_position_embedding is source-compatible with
 * include/ppl/kernel/llm/cuda/pmx/rotary_position_embedding.h:54-76 of the reference (same
 * namespace and argument list, hipStream_t for cudaStream_t).  rope_scaling carries three distinct
 * values here; the reference header defines NONE, LINEAR and DYNAMIC all as 0 (lines 27-31), which
 * makes its linear and dynamic branches unreachable.
 *
 * dynamic_batching_rotary_position_embedding_kv_cache has no counterpart in the reference: it is the
 * rotation followed in the same kernel by forward_kvstore's quantise/append
 * (multi_head_cache_attention/kernel.cu:2013-2057) of the rotated key and of the value rows.
 */
#ifndef PMX_HIP_ROTARY_POSITION_EMBEDDING_H_
#define PMX_HIP_ROTARY_POSITION_EMBEDDING_H_

#include <hip/hip_runtime_api.h>

#include <cstdint>

#include "pmx_hip/ppl_common_compat.h"

namespace ppl { namespace kernel { namespace llm { namespace cuda { namespace pmx {

typedef int32_t rope_scaling_t;

struct rope_scaling {
    static const rope_scaling_t NONE = 0;
    static const rope_scaling_t LINEAR = 1;
    static const rope_scaling_t DYNAMIC = 2;
};

PMXHIP_CXX_API ppl::common::RetCode dynamic_batching_rotary_position_embedding(
    hipStream_t stream,
    const ppl::common::TensorShape* query_shape,
    const void* query, // (seqstarts[-1], ..., head_dim), dim[1] is the leading dim of heads
    const ppl::common::TensorShape* key_shape,
    const void* key,
    const void* start_pos,
    const void* seqstarts,
    const float theta,
    const int32_t bypass_key,
    const int64_t rotary_dim,
    const int64_t batch,
    const int64_t num_heads,
    const int64_t num_key_heads,
    const int64_t max_seqlen,
    const int64_t max_position_embeddings,
    const rope_scaling_t scaling_type,
    const float scaling_factor,
    const ppl::common::TensorShape* rotated_query_shape,
    void* rotated_query,
    const ppl::common::TensorShape* rotated_key_shape,
    void* rotated_key);

// The same, then the quantise/append of the rotated key and of current_value into the int8 cache;
// rotated_key may be nullptr.  The trailing arguments are forward_kvstore's.
PMXHIP_CXX_API ppl::common::RetCode dynamic_batching_rotary_position_embedding_kv_cache(
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
    void* cache, void* scale);

}}}}} // namespace ppl::kernel::llm::cuda::pmx

#endif // PMX_HIP_ROTARY_POSITION_EMBEDDING_H_
