/*
 * The output projection that follows the cache attention, on one GPU.
 *
 * Mirrors ppl::kernel::llm::cuda::pmx::row_parallel_linear
 * (include/ppl/kernel/llm/cuda/pmx/row_parallel_linear.h:28-46 of the reference): the same argument names, order
 * and meaning, without the arguments that belong to cuBLASLt and NCCL -- cublaslt_handle, algo, nccl_param,
 * split_buffer.  A call site drops those four arguments; this build runs on one GPU, which is the reference's
 * nccl_param->size == 1 path: one GEMM, bias added, no all-reduce (row_parallel_linear.cu:61-97).  The
 * reference's cublas_workspace_size / cublas_workspace pair is kept as workspace_size / workspace: the caller's
 * scratch for the float32 partial tiles of a k-split (row_parallel_linear_workspace_size says how much serves a
 * shape; a null workspace is allowed and only costs time at decode sizes).
 *   input  (M, K) half, M = product of all but the last dimension of input_shape
 *   weight (N, K) half
 *   bias   (N) half or nullptr
 *   output (M, N) half
 * input_is_parallel = false is rejected with RC_UNSUPPORTED, as in the reference (row_parallel_linear.cu:46-49).
 */
#ifndef PMX_HIP_ROW_PARALLEL_LINEAR_H_
#define PMX_HIP_ROW_PARALLEL_LINEAR_H_

#include <hip/hip_runtime_api.h>

#include <cstdint>

#include "pmx_hip/ppl_common_compat.h"

namespace ppl { namespace kernel { namespace llm { namespace cuda { namespace pmx {

PMXHIP_CXX_API ppl::common::RetCode row_parallel_linear(
    const hipStream_t stream,
    const ppl::common::TensorShape* input_shape,
    const void* input,
    const ppl::common::TensorShape* weight_shape,
    const void* weight,
    const ppl::common::TensorShape* bias_shape,
    const void* bias,
    const int64_t in_features,
    const int64_t out_features,
    const bool input_is_parallel,
    const int64_t workspace_size,
    void* workspace,
    const ppl::common::TensorShape* output_shape,
    void* output);

// bytes of workspace that serve M rows of in_features -> out_features on the current device (0 = none needed)
PMXHIP_CXX_API int64_t row_parallel_linear_workspace_size(const int64_t m, const int64_t in_features, const int64_t out_features);

}}}}} // namespace ppl::kernel::llm::cuda::pmx

#endif // PMX_HIP_ROW_PARALLEL_LINEAR_H_
