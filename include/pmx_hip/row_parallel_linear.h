/*
 * The output projection that follows the cache attention, on one GPU.
 *
 * Mirrors ppl::kernel::llm::cuda::pmx::row_parallel_linear
 * (include/ppl/kernel/llm/cuda/pmx/row_parallel_linear.h:28-46 of the reference).  The first overload has the
 * reference's argument list, name for name and in its order (cudaStream_t reads hipStream_t): a call site compiles
 * after the include switch.  cublaslt_handle, algo and split_buffer are taken and ignored; nccl_param may be null
 * (one rank); a communicator of more than one rank is refused with RC_UNSUPPORTED: this build runs on one GPU,
 * which is the reference's nccl_param->size == 1 path: one GEMM, bias added, no all-reduce
 * (row_parallel_linear.cu:61-97).  The second overload is the same call without those four arguments.  The
 * reference's cublas_workspace_size / cublas_workspace pair is the caller's scratch for the float32 partial tiles
 * of a k-split (row_parallel_linear_workspace_size says how much serves a shape; a null workspace is allowed and
 * only costs time at decode sizes).
 *   input  (M, K) half, M = product of all but the last dimension of input_shape
 *   weight (N, K) half
 *   bias   (N) half or nullptr
 *   output (M, N) half
 * input_is_parallel = false is rejected with RC_UNSUPPORTED, as in the reference (row_parallel_linear.cu:46-49).
 * use_vendor_gemm (no counterpart in the reference, default false): row counts from 384 on go to hipBLASLt where it
 * can be loaded (c_api.h, PMXHIP_LINEAR_VENDOR_GEMM); by default this library's own kernels serve every row count.
 */
#ifndef PMX_HIP_ROW_PARALLEL_LINEAR_H_
#define PMX_HIP_ROW_PARALLEL_LINEAR_H_

#include <hip/hip_runtime_api.h>

#include <cstdint>

#include "pmx_hip/ppl_common_compat.h"

namespace ppl { namespace kernel { namespace llm { namespace cuda { namespace pmx {

PMXHIP_CXX_API ppl::common::RetCode row_parallel_linear(
    const hipStream_t stream,
    const cublasLtHandle_t& cublaslt_handle,
    const cublasLtMatmulAlgo_t* algo,
    const ppl::common::TensorShape* input_shape,
    const void* input,
    const ppl::common::TensorShape* weight_shape,
    const void* weight,
    const ppl::common::TensorShape* bias_shape,
    const void* bias,
    const int64_t in_features,
    const int64_t out_features,
    const ppl::common::NcclParam* nccl_param,
    const bool input_is_parallel,
    void* split_buffer,
    const int64_t cublas_workspace_size,
    void* cublas_workspace,
    const ppl::common::TensorShape* output_shape,
    void* output,
    const bool use_vendor_gemm = false);

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
    void* output,
    const bool use_vendor_gemm = false);

// bytes of workspace that serve M rows of in_features -> out_features on the current device (0 = none needed)
PMXHIP_CXX_API int64_t row_parallel_linear_workspace_size(const int64_t m, const int64_t in_features, const int64_t out_features,
                                                          const bool use_vendor_gemm = false);

}}}}} // namespace ppl::kernel::llm::cuda::pmx

#endif // PMX_HIP_ROW_PARALLEL_LINEAR_H_
