/*
 * key_value_cache: the quantise/append step as a free function, under the name
 * the serving stack's KeyValueCache operator uses.  In the reference tree this
 * step has no free function; it is
 * dynamic_batching_multi_head_cache_attention::forward_kvstore
 * (src/ppl/kernel/llm/cuda/pmx/multi_head_cache_attention/kernel.cu:2013-2057)
 * over dynamic_batching_kv_cache_quantize_kernel_param (kernel.cu:64-84), whose
 * argument list this function takes.
 */
#ifndef PMX_HIP_KEY_VALUE_CACHE_H_
#define PMX_HIP_KEY_VALUE_CACHE_H_

#include <hip/hip_runtime_api.h>

#include <cstdint>

#include "pmx_hip/ppl_common_compat.h"

namespace ppl { namespace kernel { namespace llm { namespace cuda { namespace pmx {

PMXHIP_CXX_API ppl::common::RetCode dynamic_batching_key_value_cache(
    const hipStream_t stream,
    const ppl::common::TensorShape* current_key_shape,
    const void* current_key, // half (S, KVH, D)
    const ppl::common::TensorShape* current_value_shape,
    const void* current_value, // half (S, KVH, D)
    const void* seqstarts, // int64 (B + 1)
    const void* cachestarts, // int64 (B) or (B, MaxP)
    const void* start_pos, // int64 (B)
    const int64_t batch,
    const int64_t max_seqlen,
    const int64_t num_layer,
    const int64_t layer_idx,
    const int64_t num_kv_heads,
    const int64_t head_dim,
    const int32_t cache_mode,
    const int64_t page_size,
    const int64_t cache_stride_s,
    const int64_t cache_stride_l,
    const int64_t cache_stride_h,
    const int64_t cache_stride_kv,
    const int64_t cachestarts_stride_b,
    void* cache, // int8
    void* scale); // half

}}}}} // namespace ppl::kernel::llm::cuda::pmx

#endif // PMX_HIP_KEY_VALUE_CACHE_H_
