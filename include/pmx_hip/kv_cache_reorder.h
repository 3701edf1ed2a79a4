/*
 * kv_cache_reorder / kv_cache_invert_reorder on MI355X: whole int8 KV pages and their scales
 * gathered into, or scattered from, a contiguous outer buffer (page swap, migration).
 *
 * Source-compatible with include/ppl/kernel/llm/cuda/pmx/kv_cache_reorder.h:25-74 of the
 * reference: same namespace, same `Stride` fields in the same order, same argument lists with
 * hipStream_t in place of cudaStream_t.  All strides are byte strides; addressing is described
 * at pmxhip_kv_cache_reorder in pmx_hip/c_api.h.
 */
#ifndef PMX_HIP_KV_CACHE_REORDER_H_
#define PMX_HIP_KV_CACHE_REORDER_H_

#include <hip/hip_runtime_api.h>

#include <cstdint>

#include "pmx_hip/ppl_common_compat.h"

namespace ppl { namespace kernel { namespace llm { namespace cuda { namespace pmx {

struct Stride {
    int p_stride_cache;
    int l_stride_cache;
    int kv_stride_cache;
    int h_stride_cache;
    int t_stride_cache;
    int d_stride_cache;

    int p_stride_scale;
    int l_stride_scale;
    int kv_stride_scale;
    int h_stride_scale;
    int t_stride_scale;
    int d_stride_scale;
};

PMXHIP_CXX_API ppl::common::RetCode kv_cache_reorder(
    hipStream_t stream,
    const void* kv_cache,
    const void* kv_scale,
    const void* page_ids, // int64 (page_nums), device
    const Stride& src_stride,
    const Stride& dst_stride,
    int64_t page_nums,
    int64_t layers,
    int64_t kv_heads,
    int64_t tokens,
    int64_t head_dim,
    int64_t group_size,
    int64_t tp_rank,
    int64_t tp_size,
    void* outer_mem);

PMXHIP_CXX_API ppl::common::RetCode kv_cache_invert_reorder(
    hipStream_t stream,
    const void* outer_mem,
    const void* page_ids,
    const Stride& src_stride,
    const Stride& dst_stride,
    int64_t page_nums,
    int64_t layers,
    int64_t kv_heads,
    int64_t tokens,
    int64_t head_dim,
    int64_t group_size,
    int64_t tp_rank,
    int64_t tp_size,
    void* kv_cache,
    void* kv_scale);

}}}}} // namespace ppl::kernel::llm::cuda::pmx

#endif // PMX_HIP_KV_CACHE_REORDER_H_
