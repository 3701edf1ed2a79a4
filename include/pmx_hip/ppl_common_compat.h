/*
 * Minimal stand-ins for the ppl.common types the operator interface names.
 * ppl.common is an external dependency of the reference (cmake/deps.cmake:90)
 * and is not in its tree; only what
 * include/ppl/kernel/llm/cuda/pmx/multi_head_cache_attention.h and
 * src/ppl/kernel/llm/cuda/pmx/multi_head_cache_attention/utils.cu:68-131,269
 * touch is provided: RetCode, datatype_t, and TensorShape's GetDim /
 * GetDimCount / GetDataType / CalcElementsExcludingPadding; and, for the argument list of
 * include/ppl/kernel/llm/cuda/pmx/row_parallel_linear.h:28-46, ppl::common::NcclParam (rank, size, communicator)
 * and the two cuBLASLt types it names as opaque stand-ins (PMX_HIP_HAVE_BLASLT_TYPES: the call site brings its own).
 * When building inside a tree that has the real ppl.common, define
 * PMX_HIP_USE_PPL_COMMON and these are taken from there instead.
 */
#ifndef PMX_HIP_PPL_COMMON_COMPAT_H_
#define PMX_HIP_PPL_COMMON_COMPAT_H_

/* libpmx_hip.so is built with hidden visibility; the operator class and the free functions of the C++ interface
 * are exported explicitly so that a call site links against the library as it links against the reference's. */
#if defined(__GNUC__)
#define PMXHIP_CXX_API __attribute__((visibility("default")))
#else
#define PMXHIP_CXX_API
#endif

#ifdef PMX_HIP_USE_PPL_COMMON
#include "ppl/common/retcode.h"
#include "ppl/common/tensor_shape.h"
#else

#include <cstdint>
#include <initializer_list>

namespace ppl { namespace common {

typedef uint32_t RetCode;
enum {
    RC_SUCCESS = 0,
    RC_OTHER_ERROR = 1,
    RC_UNSUPPORTED = 2,
    RC_OUT_OF_MEMORY = 3,
    RC_INVALID_VALUE = 4,
};

typedef uint32_t datatype_t;
enum {
    DATATYPE_UNKNOWN = 0,
    DATATYPE_FLOAT16 = 5,
    DATATYPE_FLOAT32 = 6,
    DATATYPE_INT8 = 10,
    DATATYPE_INT64 = 13,
};

class TensorShape final {
public:
    static constexpr uint32_t kMaxDims = 8;

    TensorShape() : dim_count_(0), data_type_(DATATYPE_UNKNOWN) {
        for (uint32_t i = 0; i < kMaxDims; ++i) dims_[i] = 0;
    }
    TensorShape(datatype_t dt, std::initializer_list<int64_t> dims) : TensorShape() {
        data_type_ = dt;
        for (int64_t d : dims) {
            if (dim_count_ < kMaxDims) dims_[dim_count_++] = d;
        }
    }

    void SetDataType(datatype_t dt) { data_type_ = dt; }
    datatype_t GetDataType() const { return data_type_; }

    void SetDimCount(uint32_t n) { dim_count_ = n < kMaxDims ? n : kMaxDims; }
    uint32_t GetDimCount() const { return dim_count_; }

    void SetDim(uint32_t i, int64_t v) { if (i < kMaxDims) dims_[i] = v; }
    int64_t GetDim(uint32_t i) const { return i < kMaxDims ? dims_[i] : 0; }

    uint64_t CalcElementsExcludingPadding() const {
        if (dim_count_ == 0) return 0;
        uint64_t n = 1;
        for (uint32_t i = 0; i < dim_count_; ++i) n *= (uint64_t)dims_[i];
        return n;
    }

private:
    uint32_t dim_count_;
    datatype_t data_type_;
    int64_t dims_[kMaxDims];
};

// ppl/common/cuda/nccl_utils.h: what row_parallel_linear reads of it is `size` (row_parallel_linear.cu:83)
struct NcclParam {
    int rank = 0;
    int size = 1;
    void* nccl_comm = nullptr;
};

}} // namespace ppl::common

#endif // PMX_HIP_USE_PPL_COMMON

/* The GEMM handle and algorithm of the reference's row_parallel_linear: this build takes and ignores them (its
 * own kernels, or hipBLASLt through a handle of its own), so that a call site keeps its argument list. */
#ifndef PMX_HIP_HAVE_BLASLT_TYPES
struct pmxhip_opaque_blaslt_context;
typedef pmxhip_opaque_blaslt_context* cublasLtHandle_t;
struct cublasLtMatmulAlgo_t {
    uint64_t data[8];
};
#endif
#endif // PMX_HIP_PPL_COMMON_COMPAT_H_
