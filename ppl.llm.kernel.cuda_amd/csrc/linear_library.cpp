// Output projection with many rows (a prefill chunk's thousands of query rows): a compute-bound GEMM, which is what
// the vendor's library is for -- the reference makes the same choice (one cublasLt GEMM,
// src/ppl/kernel/llm/cuda/pmx/row_parallel_linear.cu:57-81).  hipBLASLt is loaded on first use with dlopen, so the
// library has no link-time dependency on it; where it is absent (or refuses the shape) the caller runs this
// build's own kernels, which are made for decode-sized row counts.
// Host only.
#include <dlfcn.h>

#include <map>
#include <mutex>
#include <tuple>

#include <hipblaslt/hipblaslt.h>

#include "launch_params.h"

namespace pmxhip {

namespace {

struct Api {
    decltype(&hipblasLtCreate) create = nullptr;
    decltype(&hipblasLtMatrixLayoutCreate) layout_create = nullptr;
    decltype(&hipblasLtMatrixLayoutDestroy) layout_destroy = nullptr;
    decltype(&hipblasLtMatmulDescCreate) desc_create = nullptr;
    decltype(&hipblasLtMatmulDescDestroy) desc_destroy = nullptr;
    decltype(&hipblasLtMatmulDescSetAttribute) desc_set = nullptr;
    decltype(&hipblasLtMatmulPreferenceCreate) pref_create = nullptr;
    decltype(&hipblasLtMatmulPreferenceDestroy) pref_destroy = nullptr;
    decltype(&hipblasLtMatmulPreferenceSetAttribute) pref_set = nullptr;
    decltype(&hipblasLtMatmulAlgoGetHeuristic) heuristic = nullptr;
    decltype(&hipblasLtMatmul) matmul = nullptr;
    bool ok = false;
};

const Api& api()
{
    static const Api a = [] {
        Api r;
        void* lib = dlopen("libhipblaslt.so", RTLD_NOW | RTLD_LOCAL);
        if (!lib) lib = dlopen("libhipblaslt.so.1", RTLD_NOW | RTLD_LOCAL);
        if (!lib) return r;
        auto sym = [&](const char* name) { return dlsym(lib, name); };
        r.create = (decltype(r.create))sym("hipblasLtCreate");
        r.layout_create = (decltype(r.layout_create))sym("hipblasLtMatrixLayoutCreate");
        r.layout_destroy = (decltype(r.layout_destroy))sym("hipblasLtMatrixLayoutDestroy");
        r.desc_create = (decltype(r.desc_create))sym("hipblasLtMatmulDescCreate");
        r.desc_destroy = (decltype(r.desc_destroy))sym("hipblasLtMatmulDescDestroy");
        r.desc_set = (decltype(r.desc_set))sym("hipblasLtMatmulDescSetAttribute");
        r.pref_create = (decltype(r.pref_create))sym("hipblasLtMatmulPreferenceCreate");
        r.pref_destroy = (decltype(r.pref_destroy))sym("hipblasLtMatmulPreferenceDestroy");
        r.pref_set = (decltype(r.pref_set))sym("hipblasLtMatmulPreferenceSetAttribute");
        r.heuristic = (decltype(r.heuristic))sym("hipblasLtMatmulAlgoGetHeuristic");
        r.matmul = (decltype(r.matmul))sym("hipblasLtMatmul");
        r.ok = r.create && r.layout_create && r.layout_destroy && r.desc_create && r.desc_destroy && r.desc_set &&
               r.pref_create && r.pref_destroy && r.pref_set && r.heuristic && r.matmul;
        return r;
    }();
    return a;
}

std::mutex g_mutex;
std::map<int, hipblasLtHandle_t> g_handles; // per device
// the algorithm the library's heuristic picked for a problem: asked once per (device, shape, strides, bias, workspace)
using Key = std::tuple<int, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, bool, int64_t>;
std::map<Key, hipblasLtMatmulHeuristicResult_t> g_algos;

// the device's handle; created outside stream captures only (creation allocates)
int handle_for(int device, hipStream_t stream, hipblasLtHandle_t* out)
{
    std::lock_guard<std::mutex> lock(g_mutex);
    auto it = g_handles.find(device);
    if (it != g_handles.end()) {
        *out = it->second;
        return kLaunchOk;
    }
    hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &st) != hipSuccess || st != hipStreamCaptureStatusNone) {
        (void)hipGetLastError();
        return kLaunchNeedsWarmup;
    }
    hipblasLtHandle_t h = nullptr;
    if (api().create(&h) != HIPBLAS_STATUS_SUCCESS || !h) return kLaunchNoKernel;
    g_handles[device] = h;
    *out = h;
    return kLaunchOk;
}

} // namespace

bool linear_library_available() { return api().ok; }

int init_linear_library(int device)
{
    if (!api().ok) return kLaunchOk; // nothing to set up: the caller's own kernels serve every shape
    hipblasLtHandle_t h = nullptr;
    const int rc = handle_for(device, nullptr, &h);
    return rc == kLaunchNoKernel ? kLaunchOk : rc;
}

// output(M, N) = input(M, K) weight(N, K)^T + bias, row-major halves, float accumulation.  In the library's
// column-major terms: D (N x M, ld output_stride) = A^T B + bias with A = weight as K x N (ld weight_stride) and
// B = input as K x M (ld input_stride); the bias vector runs along D's rows.
// Returns kLaunchNoKernel when the library is absent or has no algorithm for the problem within the workspace.
int launch_linear_library(const LinearLaunch& a, int device, void* workspace, int64_t workspace_bytes, hipStream_t stream)
{
    const Api& f = api();
    if (!f.ok) return kLaunchNoKernel;
    hipblasLtHandle_t handle = nullptr;
    if (int rc = handle_for(device, stream, &handle)) return rc;
    if (!workspace || workspace_bytes < 0) workspace_bytes = 0;

    hipblasLtMatmulDesc_t desc = nullptr;
    hipblasLtMatrixLayout_t la = nullptr, lb = nullptr, ld = nullptr;
    hipblasLtMatmulPreference_t pref = nullptr;
    int rc = kLaunchNoKernel;
    do {
        if (f.desc_create(&desc, HIPBLAS_COMPUTE_32F, HIP_R_32F) != HIPBLAS_STATUS_SUCCESS) break;
        const int32_t op_t = HIPBLAS_OP_T, op_n = HIPBLAS_OP_N;
        if (f.desc_set(desc, HIPBLASLT_MATMUL_DESC_TRANSA, &op_t, sizeof(op_t)) != HIPBLAS_STATUS_SUCCESS) break;
        if (f.desc_set(desc, HIPBLASLT_MATMUL_DESC_TRANSB, &op_n, sizeof(op_n)) != HIPBLAS_STATUS_SUCCESS) break;
        if (a.bias) {
            const uint32_t epilogue = HIPBLASLT_EPILOGUE_BIAS;
            const int32_t bias_type = HIP_R_16F;
            const void* bias = a.bias;
            if (f.desc_set(desc, HIPBLASLT_MATMUL_DESC_EPILOGUE, &epilogue, sizeof(epilogue)) != HIPBLAS_STATUS_SUCCESS) break;
            if (f.desc_set(desc, HIPBLASLT_MATMUL_DESC_BIAS_DATA_TYPE, &bias_type, sizeof(bias_type)) != HIPBLAS_STATUS_SUCCESS) break;
            if (f.desc_set(desc, HIPBLASLT_MATMUL_DESC_BIAS_POINTER, &bias, sizeof(bias)) != HIPBLAS_STATUS_SUCCESS) break;
        }
        if (f.layout_create(&la, HIP_R_16F, (uint64_t)a.k, (uint64_t)a.n, a.weight_stride) != HIPBLAS_STATUS_SUCCESS) break;
        if (f.layout_create(&lb, HIP_R_16F, (uint64_t)a.k, (uint64_t)a.m, a.input_stride) != HIPBLAS_STATUS_SUCCESS) break;
        if (f.layout_create(&ld, HIP_R_16F, (uint64_t)a.n, (uint64_t)a.m, a.output_stride) != HIPBLAS_STATUS_SUCCESS) break;

        const Key key{device, a.m, a.n, a.k, a.input_stride, a.weight_stride, a.output_stride, a.bias != nullptr, workspace_bytes};
        hipblasLtMatmulHeuristicResult_t chosen{};
        bool have = false;
        {
            std::lock_guard<std::mutex> lock(g_mutex);
            auto it = g_algos.find(key);
            if (it != g_algos.end()) {
                chosen = it->second;
                have = true;
            }
        }
        if (!have) {
            if (f.pref_create(&pref) != HIPBLAS_STATUS_SUCCESS) break;
            const uint64_t max_ws = (uint64_t)workspace_bytes;
            if (f.pref_set(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &max_ws, sizeof(max_ws)) != HIPBLAS_STATUS_SUCCESS) break;
            // the library's candidates in its order of preference: the first that fits the caller's workspace (its
            // first choice for tall problems splits k over workgroups and wants tens of megabytes)
            constexpr int kCandidates = 16;
            hipblasLtMatmulHeuristicResult_t cand[kCandidates];
            int found = 0;
            if (f.heuristic(handle, desc, la, lb, ld, ld, pref, kCandidates, cand, &found) != HIPBLAS_STATUS_SUCCESS) break;
            for (int i = 0; i < found && !have; ++i) {
                if (cand[i].state == HIPBLAS_STATUS_SUCCESS && (int64_t)cand[i].workspaceSize <= workspace_bytes) {
                    chosen = cand[i];
                    have = true;
                }
            }
            if (!have) break;
            std::lock_guard<std::mutex> lock(g_mutex);
            g_algos[key] = chosen;
        }
        const float alpha = 1.f, beta = 0.f;
        if (f.matmul(handle, desc, &alpha, a.weight, la, a.input, lb, &beta, a.output, ld, a.output, ld, &chosen.algo, workspace,
                     (size_t)workspace_bytes, stream) != HIPBLAS_STATUS_SUCCESS)
            break;
        rc = kLaunchOk;
    } while (false);
    if (pref) f.pref_destroy(pref);
    if (ld) f.layout_destroy(ld);
    if (lb) f.layout_destroy(lb);
    if (la) f.layout_destroy(la);
    if (desc) f.desc_destroy(desc);
    return rc;
}

} // namespace pmxhip
