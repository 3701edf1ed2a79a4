// Host side of the C ABI: argument checks, the split plan, and kernel launches.
// No allocation, no synchronisation; errors are reported by return code plus a
// thread-local message (pmxhip_last_error).  The one exception is opt-in: the vendor GEMM route of
// pmxhip_row_parallel_linear_ex (PMXHIP_LINEAR_VENDOR_GEMM), whose library allocates on the host.
#include "pmx_hip/c_api.h"

#include <hip/hip_runtime.h>

#include <atomic>
#include <cstdarg>
#include <cstdio>
#include <cstring>

#include "launch_params.h"

// ---- scratch of the entry point that allocates nothing (pmxhip_decode_attention_static) ----
// Split-KV pieces of one decode step: float32 partial outputs and (max, exp-sum) pairs, the same layout the
// caller's workspace has in pmxhip_decode_attention.  One array per GPU, resident until the process ends.
// In host code the array's name is only a handle for hipGetSymbolAddress; every use of the memory goes through
// the per-device pointer resolved below.
constexpr int64_t kStaticScratchBytes = PMXHIP_STATIC_WORKSPACE_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

namespace {

thread_local char g_last_error[512] = "";
thread_local bool g_quiet = false; // a check whose failure only selects another route: no message on stderr

int fail(int code, const char* fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
    va_end(ap);
    if (!g_quiet) fprintf(stderr, "[pmx_hip] error: %s\n", g_last_error);
    return code;
}

bool head_dim_supported(int64_t d) { return d == 64 || d == 96 || d == 128 || d == 256; }

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

int check_cache_layout(const char* who, int32_t cache_mode, int64_t page_size, int64_t s, int64_t l, int64_t h,
                       int64_t kv, int64_t multiple)
{
    if (cache_mode != 0 && cache_mode != 1) return fail(PMXHIP_UNSUPPORTED, "%s: invalid cache_mode %d", who, cache_mode);
    if (cache_mode == 1 && page_size != PMXHIP_PAGE_SIZE)
        return fail(PMXHIP_UNSUPPORTED, "%s: cache_mode 1 needs page_size == %d, got %lld", who, PMXHIP_PAGE_SIZE,
                    (long long)page_size);
    if (s % multiple || l % multiple || h % multiple || kv % multiple)
        return fail(PMXHIP_UNSUPPORTED, "%s: cache strides must be multiples of %lld (s=%lld l=%lld h=%lld kv=%lld)", who,
                    (long long)multiple, (long long)s, (long long)l, (long long)h, (long long)kv);
    return PMXHIP_SUCCESS;
}

int launch_status(const char* who)
{
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(PMXHIP_OTHER_ERROR, "%s: launch failed: %s", who, hipGetErrorString(e));
    return PMXHIP_SUCCESS;
}

int launch_result(const char* who, int launch_rc)
{
    if (launch_rc == pmxhip::kLaunchNoKernel) return fail(PMXHIP_UNSUPPORTED, "%s: no kernel for this shape", who);
    if (launch_rc == pmxhip::kLaunchNeedsWarmup)
        return fail(PMXHIP_OTHER_ERROR,
                    "%s: the first launch of this kernel in the process came while the stream is being captured; "
                    "call pmxhip_init() (or run one step outside the capture) first", who);
    return launch_status(who);
}

// Compute units of the current device, looked up once per device.
int current_compute_units()
{
    constexpr int kMaxDevices = 64;
    static std::atomic<int> cached[kMaxDevices];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return 0;
    int cus = cached[dev].load(std::memory_order_relaxed);
    if (cus == 0) {
        if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 0;
        cached[dev].store(cus, std::memory_order_relaxed);
    }
    return cus;
}

constexpr int kScratchDevices = 64;
std::atomic<void*> g_scratch_ptr[kScratchDevices];

// The device address of `scratch` on the current device; resolved on first use per device (never under capture).
int static_scratch(const char* who, pmxhip_stream_t stream, void** out)
{
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kScratchDevices)
        return fail(PMXHIP_OTHER_ERROR, "%s: no current device", who);
    void* ptr = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (!ptr) {
        hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing(stream, &st) != hipSuccess || st != hipStreamCaptureStatusNone) {
            (void)hipGetLastError();
            return fail(PMXHIP_OTHER_ERROR, "%s: first call on this device under stream capture; call pmxhip_init() first", who);
        }
        const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !ptr)
            return fail(PMXHIP_OTHER_ERROR, "%s: hipGetSymbolAddress failed: %s", who, hipGetErrorString(e));
        g_scratch_ptr[dev].store(ptr, std::memory_order_release);
    }
    *out = ptr;
    return PMXHIP_SUCCESS;
}

} // namespace

extern "C" {

const char* pmxhip_version(void) { return "pmx_hip 0.2 (gfx950)"; }

int pmxhip_init(void)
{
    if (pmxhip::init_decode_kernels() != 0 || pmxhip::init_prefill_kernels() != 0) {
        const hipError_t e = hipGetLastError();
        return fail(PMXHIP_OTHER_ERROR, "init: hipFuncSetAttribute failed: %s", hipGetErrorString(e));
    }
    void* ptr = nullptr;
    if (int rc = static_scratch("init", nullptr, &ptr)) return rc;
    (void)current_compute_units();
    return PMXHIP_SUCCESS;
}

int pmxhip_init_vendor_gemm(void)
{
    int device = 0;
    if (hipGetDevice(&device) != hipSuccess) return fail(PMXHIP_OTHER_ERROR, "init_vendor_gemm: no current device");
    if (!pmxhip::linear_library_available() || pmxhip::init_linear_library(device) != 0)
        return fail(PMXHIP_UNSUPPORTED, "init_vendor_gemm: hipBLASLt could not be loaded or gave no handle");
    return PMXHIP_SUCCESS;
}

const char* pmxhip_last_error(void) { return g_last_error; }

int pmxhip_kv_cache_quantize(const pmxhip_kvstore_params* p, pmxhip_stream_t stream)
{
    if (!p) return fail(PMXHIP_INVALID_VALUE, "kv_cache_quantize: null params");
    if (p->head_dim <= 0 || p->head_dim % 8 != 0) // kernel.cu:2040-2043
        return fail(PMXHIP_UNSUPPORTED, "kv_cache_quantize: head_dim must be aligned with 8, currently get %lld",
                    (long long)p->head_dim);
    if (int rc = check_cache_layout("kv_cache_quantize", p->cache_mode, p->page_size, p->cache_stride_s, p->cache_stride_l,
                                    p->cache_stride_h, p->cache_stride_kv, 8))
        return rc;
    if (p->batch < 0 || p->max_seqlen < 0 || p->num_kv_heads <= 0)
        return fail(PMXHIP_INVALID_VALUE, "kv_cache_quantize: bad batch/max_seqlen/num_kv_heads");
    if (p->batch == 0 || p->max_seqlen == 0) return PMXHIP_SUCCESS;
    if (!p->current_key || !p->current_value || !p->seqstarts || !p->cachestarts || !p->start_pos || !p->cache || !p->scale)
        return fail(PMXHIP_INVALID_VALUE, "kv_cache_quantize: null device pointer");
    if (p->current_key_stride_s % 8 || p->current_value_stride_s % 8 || !aligned16(p->current_key) ||
        !aligned16(p->current_value) || (reinterpret_cast<uintptr_t>(p->cache) & 7u))
        return fail(PMXHIP_UNSUPPORTED, "kv_cache_quantize: current_key/value need 16-byte aligned rows, cache 8-byte alignment");

    pmxhip::QuantLaunch a{};
    a.current_key = p->current_key;
    a.current_value = p->current_value;
    a.seqstarts = p->seqstarts;
    a.cachestarts = p->cachestarts;
    a.start_pos = p->start_pos;
    a.cache = static_cast<int8_t*>(p->cache);
    a.scale = p->scale;
    a.batch = p->batch;
    a.layer_idx = p->layer_idx;
    a.num_kv_heads = (int32_t)p->num_kv_heads;
    a.head_dim = (int32_t)p->head_dim;
    a.current_key_stride_s = p->current_key_stride_s;
    a.current_value_stride_s = p->current_value_stride_s;
    a.cache_stride_s = p->cache_stride_s;
    a.cache_stride_l = p->cache_stride_l;
    a.cache_stride_h = p->cache_stride_h;
    a.cache_stride_kv = p->cache_stride_kv;
    a.cachestarts_stride_b = p->cachestarts_stride_b;
    a.max_tokens = p->batch * p->max_seqlen;
    a.cache_mode = p->cache_mode;
    return launch_result("kv_cache_quantize", pmxhip::launch_kv_quantize(a, current_compute_units(), stream));
}

int pmxhip_key_value_cache(pmxhip_stream_t stream, const void* current_key, const void* current_value,
                           const int64_t* seqstarts, const int64_t* cachestarts, const int64_t* start_pos, int64_t batch,
                           int64_t max_seqlen, int64_t num_layer, int64_t layer_idx, int64_t num_kv_heads,
                           int64_t head_dim, int32_t cache_mode, int64_t page_size, int64_t cache_stride_s,
                           int64_t cache_stride_l, int64_t cache_stride_h, int64_t cache_stride_kv,
                           int64_t cachestarts_stride_b, void* cache, void* scale)
{
    pmxhip_kvstore_params p;
    memset(&p, 0, sizeof(p));
    p.current_key = current_key;
    p.current_value = current_value;
    p.seqstarts = seqstarts;
    p.cachestarts = cachestarts;
    p.start_pos = start_pos;
    p.num_layer = num_layer;
    p.layer_idx = layer_idx;
    p.num_kv_heads = num_kv_heads;
    p.head_dim = head_dim;
    p.page_size = (int32_t)page_size;
    p.current_key_stride_s = num_kv_heads * head_dim;
    p.current_value_stride_s = num_kv_heads * head_dim;
    p.cache_stride_s = cache_stride_s;
    p.cache_stride_l = cache_stride_l;
    p.cache_stride_h = cache_stride_h;
    p.cache_stride_kv = cache_stride_kv;
    p.cachestarts_stride_b = cachestarts_stride_b;
    p.cache = cache;
    p.scale = scale;
    p.batch = batch;
    p.max_seqlen = max_seqlen;
    p.cache_mode = cache_mode;
    return pmxhip_kv_cache_quantize(&p, stream);
}

int pmxhip_decode_plan_make(int64_t decoding_batches, int64_t num_heads, int64_t num_kv_heads, int64_t head_dim,
                            int64_t max_kvlen, int32_t compute_units, int32_t num_token_ranges_hint,
                            pmxhip_decode_plan* plan)
{
    return pmxhip_decode_plan_make_kernel(decoding_batches, num_heads, num_kv_heads, head_dim, max_kvlen, compute_units,
                                          num_token_ranges_hint, PMXHIP_DECODE_KERNEL_AUTO, plan);
}

int pmxhip_decode_plan_make_kernel(int64_t decoding_batches, int64_t num_heads, int64_t num_kv_heads, int64_t head_dim,
                                   int64_t max_kvlen, int32_t compute_units, int32_t num_token_ranges_hint,
                                   int32_t kernel_request, pmxhip_decode_plan* plan)
{
    if (!plan) return fail(PMXHIP_INVALID_VALUE, "decode_plan: null plan");
    memset(plan, 0, sizeof(*plan));
    if (!head_dim_supported(head_dim))
        return fail(PMXHIP_UNSUPPORTED, "cache flash decoding attention do not support head dim %lld", (long long)head_dim);
    if (num_kv_heads <= 0 || num_heads <= 0 || num_heads % num_kv_heads != 0)
        return fail(PMXHIP_UNSUPPORTED, "only support num_heads %% num_kv_heads == 0.");
    if (num_token_ranges_hint < 0) return fail(PMXHIP_INVALID_VALUE, "decode_plan: negative range hint");
    if (kernel_request < PMXHIP_DECODE_KERNEL_AUTO || kernel_request > PMXHIP_DECODE_KERNEL_MFMA32)
        return fail(PMXHIP_INVALID_VALUE, "decode_plan: unknown kernel request %d", kernel_request);
    pmxhip::DecodeChoice c;
    if (!pmxhip::decode_choose(head_dim, num_heads, num_kv_heads, kernel_request, &c))
        return fail(PMXHIP_UNSUPPORTED, "decode_plan: kernel %d (%s) does not serve %lld query / %lld kv heads of %lld channels",
                    kernel_request, pmxhip::decode_kernel_name(kernel_request), (long long)num_heads, (long long)num_kv_heads,
                    (long long)head_dim);
    const int min_tokens = pmxhip::decode_min_tokens_per_range(c.wg_tokens);

    int64_t ranges = num_token_ranges_hint;
    if (ranges == 0) {
        const int64_t groups = ((num_kv_heads + c.kv_heads_per_group - 1) / c.kv_heads_per_group) * c.num_passes;
        int cus = compute_units > 0 ? compute_units : current_compute_units();
        if (cus <= 0) return fail(PMXHIP_INVALID_VALUE, "decode_plan: compute_units not given and no current device");
        // as many ranges as the kernel wants workgroups per CU for a long stream (decode_select.cpp: the quad kernel
        // one wave per SIMD, the others two; more, smaller workgroups where a wave serves one or two kv heads)
        const int64_t long_slots = (int64_t)cus * c.wgs_per_cu;
        const int64_t slots = (int64_t)cus * c.wgs_per_cu_short; // what the rules for short batches below count with
        ranges = (long_slots + groups - 1) / groups;
        // A short batch: ranges of about 128 tokens (twice the smallest) where those still fill half of the slots,
        // shorter ones -- down to the smallest -- only to get that far: a piece has a fixed cost, and an idle CU costs more.
        const int64_t max_tokens = decoding_batches * (max_kvlen > 0 ? max_kvlen : 1);
        const int64_t comfortable = 2 * (int64_t)min_tokens;
        const int64_t useful = (max_tokens + comfortable - 1) / comfortable;
        if (ranges > useful) {
            ranges = useful;
            const int64_t half = slots / 2 / groups > 1 ? slots / 2 / groups : 1;
            if (ranges < half) {
                const int64_t finer = (max_tokens + min_tokens - 1) / min_tokens;
                ranges = half < finer ? half : finer;
            }
            // a step of a few sequences: below a workgroup per two CUs the ranges go down to the kernel's floor
            const int64_t sparse = cus / 2 / groups > 1 ? cus / 2 / groups : 1;
            if (ranges < sparse) {
                const int floor_tokens = pmxhip::decode_floor_tokens_per_range(c.wg_tokens);
                const int64_t finest = (max_tokens + floor_tokens - 1) / floor_tokens;
                ranges = sparse < finest ? sparse : finest;
            }
        }
        if (ranges < 1) ranges = 1;
    }
    plan->num_token_ranges = (int32_t)ranges;
    plan->kv_heads_per_group = c.kv_heads_per_group;
    plan->q_heads_per_pass = c.q_heads_per_pass;
    plan->num_passes = c.num_passes;
    plan->kernel = c.kernel;
    if (ranges > 1) {
        const int64_t pieces = ranges + decoding_batches;
        plan->partial_out_size = pieces * num_heads * head_dim * (int64_t)sizeof(float);
        plan->partial_ml_size = pieces * num_heads * 2 * (int64_t)sizeof(float);
    }
    plan->workspace_size = plan->partial_out_size + plan->partial_ml_size;
    return PMXHIP_SUCCESS;
}

namespace {

// Checks of a decode call and the launch block it becomes.  `workspace` / `workspace_size` are the caller's
// (pmxhip_decode_attention) or the library's static array (pmxhip_decode_attention_static).
int decode_prepare(const char* who, const pmxhip_decode_params* p, void* workspace, int64_t workspace_size,
                   pmxhip::DecodeLaunch* out)
{
    if (!head_dim_supported(p->head_dim))
        return fail(PMXHIP_UNSUPPORTED, "cache flash decoding attention do not support head dim %lld", (long long)p->head_dim);
    if (p->num_kv_heads <= 0 || p->num_heads % p->num_kv_heads != 0 || p->num_kv_repeats != p->num_heads / p->num_kv_heads)
        return fail(PMXHIP_UNSUPPORTED, "only support num_heads %% num_kv_heads == 0.");
    if (int rc = check_cache_layout(who, p->cache_mode, p->page_size, p->cache_stride_s, p->cache_stride_l,
                                    p->cache_stride_h, p->cache_stride_kv, 16))
        return rc;
    if (!p->query || !p->output || !p->cache || !p->scale || !p->cachestarts || !p->kvstarts)
        return fail(PMXHIP_INVALID_VALUE, "%s: null device pointer", who);
    if (!aligned16(p->query) || !aligned16(p->cache) || (reinterpret_cast<uintptr_t>(p->scale) & 3u) ||
        p->query_stride_s % 8 != 0)
        return fail(PMXHIP_UNSUPPORTED, "%s: query/cache must be 16-byte aligned, scale 4-byte aligned", who);
    if ((reinterpret_cast<uintptr_t>(p->output) & 7u) || p->output_stride_s % 4 != 0) // 8-byte stores of four halves
        return fail(PMXHIP_UNSUPPORTED, "%s: output must be 8-byte aligned with a row stride that is a multiple of 4", who);
    if (p->attn_mask && p->mask_stride_s % 8 != 0) // utils.cu:127-130
        return fail(PMXHIP_UNSUPPORTED, "last dimension of attn_mask must be aligned with 8");
    if (p->num_token_ranges <= 0) return fail(PMXHIP_INVALID_VALUE, "%s: num_token_ranges must be >= 1", who);
    if (p->kernel_request < PMXHIP_DECODE_KERNEL_AUTO || p->kernel_request > PMXHIP_DECODE_KERNEL_MFMA32)
        return fail(PMXHIP_INVALID_VALUE, "%s: unknown kernel request %d", who, p->kernel_request);

    pmxhip::DecodeLaunch a{};
    a.query = p->query;
    a.attn_mask = p->attn_mask;
    a.output = p->output;
    a.cache = p->cache;
    a.scale = p->scale;
    a.cachestarts = p->cachestarts;
    a.kvstarts = p->kvstarts;
    a.attn_scale = p->attn_scale;
    a.cache_mode = p->cache_mode;
    a.layer_idx = p->layer_idx;
    a.num_kv_repeats = p->num_kv_repeats;
    a.query_stride_s = p->query_stride_s;
    a.output_stride_s = p->output_stride_s;
    a.mask_stride_s = p->mask_stride_s;
    a.mask_stride_h = p->mask_stride_h;
    a.cache_stride_s = p->cache_stride_s;
    a.cache_stride_l = p->cache_stride_l;
    a.cache_stride_h = p->cache_stride_h;
    a.cache_stride_kv = p->cache_stride_kv;
    a.cachestarts_stride_b = p->cachestarts_stride_b;
    a.decoding_batches = p->decoding_batches;
    a.num_heads = p->num_heads;
    a.num_kv_heads = p->num_kv_heads;
    a.head_dim = (int32_t)p->head_dim;
    a.ranges = p->num_token_ranges;

    // The kernel that will run, decided once and here: by shape (or by request), then by what the quad kernel
    // needs of the buffers beyond this entry point's own checks.  Everything that depends on the kernel (the unit
    // of the range cuts above all, which the combine kernel must share) follows from this one choice.
    pmxhip::DecodeChoice c;
    if (!pmxhip::decode_choose(p->head_dim, p->num_heads, p->num_kv_heads, p->kernel_request, &c))
        return fail(PMXHIP_UNSUPPORTED, "%s: kernel %d (%s) does not serve this shape", who, p->kernel_request,
                    pmxhip::decode_kernel_name(p->kernel_request));
    if (c.kernel == pmxhip::kDecodeKernelQuad && !pmxhip::decode_quad_launch_ok(a)) {
        if (p->kernel_request == PMXHIP_DECODE_KERNEL_QUAD)
            return fail(PMXHIP_UNSUPPORTED, "%s: the quad kernel needs 16-byte aligned output rows and, with attn_mask, at "
                                            "most four query heads per kv head", who);
        pmxhip::decode_choose(p->head_dim, p->num_heads, p->num_kv_heads, pmxhip::kDecodeKernelGeneral, &c);
    }
    // ... and by the cache layout: 32-bit lane offsets against a 64-bit base per wave (decode_fit_cache_strides)
    if (!pmxhip::decode_fit_cache_strides(p->head_dim, p->num_heads, p->num_kv_heads, p->kernel_request, p->cache_stride_s,
                                          p->cache_stride_h, &c))
        return fail(PMXHIP_UNSUPPORTED,
                    "%s: cache_stride_s %lld / cache_stride_h %lld: the rows of one block of %d tokens%s must lie within 2 GiB",
                    who, (long long)p->cache_stride_s, (long long)p->cache_stride_h, c.wg_tokens,
                    c.kernel == pmxhip::kDecodeKernelQuad ? " of the two kv heads of a wave (requested quad kernel)" : "");
    a.kernel = c.kernel;
    a.kv_heads_per_group = c.kv_heads_per_group;
    a.q_heads_per_pass = c.q_heads_per_pass;
    a.num_passes = c.num_passes;
    a.wg_tokens = c.wg_tokens;
    a.min_tokens_per_range = pmxhip::decode_floor_tokens_per_range(c.wg_tokens);

    if (a.ranges > 1) {
        const int64_t pieces = (int64_t)a.ranges + p->decoding_batches;
        const int64_t out_bytes = pieces * p->num_heads * p->head_dim * (int64_t)sizeof(float);
        const int64_t ml_bytes = pieces * p->num_heads * 2 * (int64_t)sizeof(float);
        if (!workspace || workspace_size < out_bytes + ml_bytes)
            return fail(PMXHIP_INVALID_VALUE, "%s: workspace too small (%lld < %lld)", who, (long long)workspace_size,
                        (long long)(out_bytes + ml_bytes));
        if (!aligned16(workspace)) return fail(PMXHIP_INVALID_VALUE, "%s: workspace must be 16-byte aligned", who);
        a.partial_out = static_cast<float*>(workspace);
        a.partial_ml = reinterpret_cast<float*>(static_cast<char*>(workspace) + out_bytes);
    }

    *out = a;
    return PMXHIP_SUCCESS;
}

int decode_prepare_quiet(const char* who, const pmxhip_decode_params* p, void* workspace, int64_t workspace_size,
                         pmxhip::DecodeLaunch* out)
{
    g_quiet = true;
    const int rc = decode_prepare(who, p, workspace, workspace_size, out);
    g_quiet = false;
    return rc;
}

} // namespace

int pmxhip_decode_attention(const pmxhip_decode_params* p, pmxhip_stream_t stream)
{
    return pmxhip_decode_attention_stage(p, 0, stream);
}

int pmxhip_decode_attention_stage(const pmxhip_decode_params* p, int32_t stage, pmxhip_stream_t stream)
{
    if (stage < 0 || stage > 2) return fail(PMXHIP_INVALID_VALUE, "decode_attention: stage must be 0, 1 or 2");
    if (!p) return fail(PMXHIP_INVALID_VALUE, "decode_attention: null params");
    if (p->decoding_batches < 0) return fail(PMXHIP_INVALID_VALUE, "decode_attention: negative decoding_batches");
    if (p->decoding_batches == 0) return PMXHIP_SUCCESS; // kernel.cu:2084
    pmxhip::DecodeLaunch a;
    if (int rc = decode_prepare("decode_attention", p, p->workspace, p->workspace_size, &a)) return rc;
    return launch_result("decode_attention", pmxhip::launch_decode(a, stage, stream));
}

int pmxhip_decode_attention_static(const pmxhip_decode_params* p, pmxhip_stream_t stream)
{
    if (!p) return fail(PMXHIP_INVALID_VALUE, "decode_attention_static: null params");
    if (p->decoding_batches < 0) return fail(PMXHIP_INVALID_VALUE, "decode_attention_static: negative decoding_batches");
    if (p->decoding_batches == 0) return PMXHIP_SUCCESS;
    if (p->num_token_ranges > 1) {
        const double need = ((double)p->num_token_ranges + (double)p->decoding_batches) * (double)p->num_heads *
                            ((double)p->head_dim + 2.0) * sizeof(float);
        if (need > (double)kStaticScratchBytes)
            return fail(PMXHIP_INVALID_VALUE,
                        "decode_attention_static: the split-KV pieces of this call need %.0f bytes, the static workspace "
                        "holds %lld; use fewer token ranges or pmxhip_decode_attention with a workspace of your own",
                        need, (long long)kStaticScratchBytes);
    }
    void* ws = nullptr; // one range: every sequence is written as final output and no piece passes through memory
    if (p->num_token_ranges > 1)
        if (int rc = static_scratch("decode_attention_static", stream, &ws)) return rc;
    pmxhip::DecodeLaunch a;
    if (int rc = decode_prepare("decode_attention_static", p, ws, ws ? kStaticScratchBytes : 0, &a)) return rc;
    return launch_result("decode_attention_static", pmxhip::launch_decode(a, 0, stream));
}

const char* pmxhip_decode_kernel_name(const pmxhip_decode_params* p)
{
    if (!p || p->decoding_batches <= 0) return "";
    pmxhip::DecodeLaunch a;
    // the workspace plays no part in the choice; a dummy satisfies the size check
    alignas(16) static char dummy[16];
    if (decode_prepare_quiet("decode_kernel_name", p, p->workspace ? p->workspace : dummy, INT64_MAX, &a) != PMXHIP_SUCCESS) return "";
    return pmxhip::decode_kernel_name(a.kernel);
}

int pmxhip_splitkv_combine(const float* partial_out, const float* partial_ml, const int64_t* piece_begin,
                           const int64_t* piece_end, int64_t rows, int64_t head_dim, void* output,
                           pmxhip_stream_t stream)
{
    if (rows < 0 || head_dim <= 0) return fail(PMXHIP_INVALID_VALUE, "splitkv_combine: bad rows/head_dim");
    if (rows == 0) return PMXHIP_SUCCESS;
    if (!partial_out || !partial_ml || !piece_begin || !piece_end || !output)
        return fail(PMXHIP_INVALID_VALUE, "splitkv_combine: null device pointer");
    pmxhip::launch_splitkv_combine_rows(partial_out, partial_ml, piece_begin, piece_end, rows, head_dim, output, stream);
    return launch_status("splitkv_combine");
}

namespace {

// Short chunks (a few query tokens per sequence: speculative decoding's candidates, the tail of a chunked prefill)
// leave most of the tile kernel's 256 columns empty and are bound by its tile staging.  Where a kv head's (query
// position, query head) pairs fit the 32 columns of the decode step's MFMA kernel they run there instead, over token
// ranges with a combine kernel, which streams the cache at the decode rate.  That path has no mask, alibi or fp16-K/V
// form and serves head_dim 64 and 128.
constexpr int64_t kPrefillChunkColumns = 32;

bool prefill_chunk_shape(int64_t max_seqlen, int64_t num_heads, int64_t num_kv_heads, int64_t head_dim)
{
    if (head_dim != 64 && head_dim != 128) return false;
    if (num_kv_heads <= 0 || num_heads % num_kv_heads != 0 || max_seqlen <= 0) return false;
    return max_seqlen * (num_heads / num_kv_heads) <= kPrefillChunkColumns;
}

// the kernel of that path: the 16-column form where the columns fit it (head_dim 128 only), else the 32-column form
int32_t prefill_chunk_kernel(int64_t columns, int64_t head_dim)
{
    return columns <= 16 && head_dim == 128 ? PMXHIP_DECODE_KERNEL_MFMA16 : PMXHIP_DECODE_KERNEL_MFMA32;
}

// the plan of that path: a decode step of `prefill_batches` sequences whose kv heads have max_seqlen * G columns each
int prefill_chunk_plan(int64_t prefill_batches, int64_t max_seqlen, int64_t max_kvlen, int64_t num_heads, int64_t num_kv_heads,
                       int64_t head_dim, int32_t compute_units, pmxhip_decode_plan* plan)
{
    const int64_t columns = max_seqlen * (num_heads / num_kv_heads);
    return pmxhip_decode_plan_make_kernel(prefill_batches, num_kv_heads * columns, num_kv_heads, head_dim, max_kvlen,
                                          compute_units, 0, prefill_chunk_kernel(columns, head_dim), plan);
}

} // namespace

int64_t pmxhip_prefill_workspace_size(int64_t batch, int64_t decoding_batches, int64_t max_seqlen, int64_t max_kvlen,
                                      int64_t num_heads, int64_t num_kv_heads, int64_t head_dim, int32_t compute_units)
{
    const int64_t prefill_batches = batch - decoding_batches;
    if (prefill_batches <= 0 || decoding_batches < 0 || !prefill_chunk_shape(max_seqlen, num_heads, num_kv_heads, head_dim)) return 0;
    pmxhip_decode_plan plan;
    if (prefill_chunk_plan(prefill_batches, max_seqlen, max_kvlen, num_heads, num_kv_heads, head_dim, compute_units, &plan) != PMXHIP_SUCCESS)
        return 0;
    return plan.workspace_size;
}

int pmxhip_prefill_attention(const pmxhip_prefill_params* p, pmxhip_stream_t stream)
{
    if (!p) return fail(PMXHIP_INVALID_VALUE, "prefill_attention: null params");
    const int64_t prefill_batches = p->batch - p->decoding_batches;
    if (prefill_batches < 0 || p->decoding_batches < 0)
        return fail(PMXHIP_INVALID_VALUE, "prefill_attention: decoding_batches out of range");
    if (prefill_batches == 0 || p->max_seqlen == 0) return PMXHIP_SUCCESS; // kernel.cu:2130, 2214-2216
    if (p->head_dim != 64 && p->head_dim != 96 && p->head_dim != 128 && p->head_dim != 256)
        return fail(PMXHIP_UNSUPPORTED, "prefill_attention: head dim %lld not supported (64, 96, 128, 256)", (long long)p->head_dim);
    if (p->num_kv_heads <= 0 || p->num_heads % p->num_kv_heads != 0)
        return fail(PMXHIP_UNSUPPORTED, "only support num_heads %% num_kv_heads == 0.");
    const bool from_current = p->current_key != nullptr;
    if (from_current) {
        if (!p->current_value || !p->query || !p->output || !p->seqstarts)
            return fail(PMXHIP_INVALID_VALUE, "prefill_attention: null device pointer");
        if (!aligned16(p->current_key) || !aligned16(p->current_value) || p->key_stride_s % 8 != 0 || p->value_stride_s % 8 != 0 ||
            p->key_stride_s <= 0 || p->value_stride_s <= 0 || 64.0 * (double)p->key_stride_s >= 2147483648.0 ||
            64.0 * (double)p->value_stride_s >= 2147483648.0)
            return fail(PMXHIP_UNSUPPORTED, "prefill_attention: current_key/value must be 16-byte aligned with row strides that are multiples of 8");
    } else {
        if (int rc = check_cache_layout("prefill_attention", p->cache_mode, p->page_size, p->cache_stride_s, p->cache_stride_l,
                                        p->cache_stride_h, p->cache_stride_kv, 8))
            return rc;
        if (!p->query || !p->output || !p->cache || !p->scale || !p->seqstarts || !p->kvstarts || !p->cachestarts)
            return fail(PMXHIP_INVALID_VALUE, "prefill_attention: null device pointer");
        if (reinterpret_cast<uintptr_t>(p->cache) & 7u)
            return fail(PMXHIP_UNSUPPORTED, "prefill_attention: cache must be 8-byte aligned");
        // per-lane cache offsets inside a 64-token tile are 32-bit
        if (p->cache_stride_s < 0 || 64.0 * (double)p->cache_stride_s + (double)p->head_dim >= 2147483648.0)
            return fail(PMXHIP_UNSUPPORTED, "prefill_attention: cache_stride_s too large for 32-bit lane offsets");
    }
    if (!aligned16(p->query) || p->query_stride_s % 8 != 0)
        return fail(PMXHIP_UNSUPPORTED, "prefill_attention: query must be 16-byte aligned with a row stride that is a multiple of 8");
    if ((reinterpret_cast<uintptr_t>(p->output) & 7u) || p->output_stride_s % 4 != 0)
        return fail(PMXHIP_UNSUPPORTED, "prefill_attention: output must be 8-byte aligned with a row stride that is a multiple of 4");

    // short chunks on the decode step's kernels, where the shape, the inputs and the caller's workspace allow.  That
    // route computes max_seqlen query positions per sequence, so a max_seqlen that the row count of the prefill
    // sequences proves too small (more rows than sequences * max_seqlen) keeps the batch on the tile kernel, which
    // walks every row whatever the hint.
    const bool hint_covers_rows = p->prefill_query_rows <= 0 || p->prefill_query_rows <= prefill_batches * p->max_seqlen;
    if (!from_current && !p->attn_mask && !p->alibi_slopes && p->workspace && aligned16(p->workspace) && hint_covers_rows &&
        prefill_chunk_shape(p->max_seqlen, p->num_heads, p->num_kv_heads, p->head_dim)) {
        pmxhip_decode_plan plan;
        if (prefill_chunk_plan(prefill_batches, p->max_seqlen, p->max_kvlen, p->num_heads, p->num_kv_heads, p->head_dim, 0, &plan) ==
                PMXHIP_SUCCESS &&
            plan.workspace_size <= p->workspace_size && aligned16(p->cache) && !(reinterpret_cast<uintptr_t>(p->scale) & 3u) &&
            // what the decode kernels ask of the layout beyond this stage's own checks (else: the tile kernel)
            p->cache_stride_s % 16 == 0 && p->cache_stride_l % 16 == 0 && p->cache_stride_h % 16 == 0 && p->cache_stride_kv % 16 == 0 &&
            p->cache_stride_h >= 0 && p->cache_stride_s >= 0 && 32.0 * (double)p->cache_stride_s + 256.0 < 2147483648.0) {
            const int64_t g = p->num_heads / p->num_kv_heads;
            pmxhip_decode_params d;
            memset(&d, 0, sizeof(d));
            d.query = p->query;
            d.output = p->output;
            d.cache = p->cache;
            d.scale = p->scale;
            d.cachestarts = p->cachestarts + p->decoding_batches * p->cachestarts_stride_b;
            d.kvstarts = p->kvstarts + p->decoding_batches;
            d.attn_scale = p->attn_scale;
            d.layer_idx = p->layer_idx;
            d.num_kv_repeats = p->max_seqlen * g; // columns per kv head
            d.page_size = p->page_size;
            d.query_stride_s = p->query_stride_s;
            d.output_stride_s = p->output_stride_s;
            d.cache_stride_s = p->cache_stride_s;
            d.cache_stride_l = p->cache_stride_l;
            d.cache_stride_h = p->cache_stride_h;
            d.cache_stride_kv = p->cache_stride_kv;
            d.cachestarts_stride_b = p->cachestarts_stride_b;
            d.decoding_batches = prefill_batches;
            d.num_heads = p->num_kv_heads * d.num_kv_repeats;
            d.num_kv_heads = p->num_kv_heads;
            d.head_dim = p->head_dim;
            d.cache_mode = p->cache_mode;
            d.num_token_ranges = plan.num_token_ranges;
            d.workspace = p->workspace;
            d.workspace_size = p->workspace_size;
            d.kernel_request = prefill_chunk_kernel(d.num_kv_repeats, p->head_dim);
            pmxhip::DecodeLaunch c;
            // what the decode kernels refuse (an alignment, a stride) the tile kernel may still serve
            if (decode_prepare_quiet("prefill_attention", &d, d.workspace, d.workspace_size, &c) == PMXHIP_SUCCESS) {
                c.seqstarts = p->seqstarts + p->decoding_batches;
                c.chunk_q_heads = (int32_t)g;
                c.chunk_causal = p->is_causal ? 1 : 0;
                return launch_result("prefill_attention", pmxhip::launch_decode(c, 0, stream));
            }
        }
    }

    pmxhip::PrefillLaunch a{};
    a.query = p->query;
    a.output = p->output;
    a.cache = p->cache;
    a.scale = p->scale;
    a.seqstarts = p->seqstarts + p->decoding_batches;                          // kernel.cu:2131
    if (from_current) {
        a.kvstarts = a.seqstarts;                                              // kernel.cu:2196: seqstart_k = seqstart_q
        a.cachestarts = nullptr;
        a.current_key = p->current_key;
        a.current_value = p->current_value;
        a.key_stride_s = p->key_stride_s;
        a.value_stride_s = p->value_stride_s;
    } else {
        a.kvstarts = p->kvstarts + p->decoding_batches;                        // kernel.cu:2132
        a.cachestarts = p->cachestarts + p->decoding_batches * p->cachestarts_stride_b; // kernel.cu:2142
    }
    a.attn_mask = p->attn_mask;
    a.mask_stride_s = p->mask_stride_s;
    a.mask_stride_h = p->mask_stride_h;
    a.alibi_slopes = p->alibi_slopes;
    a.attn_scale = p->attn_scale;
    a.is_causal = p->is_causal;
    a.cache_mode = p->cache_mode;
    a.prefill_batches = prefill_batches;
    a.max_seqlen = p->max_seqlen;
    a.query_rows = p->prefill_query_rows > 0 ? p->prefill_query_rows : 0;
    a.layer_idx = p->layer_idx;
    a.num_heads = p->num_heads;
    a.num_kv_heads = p->num_kv_heads;
    a.head_dim = (int32_t)p->head_dim;
    a.query_stride_s = p->query_stride_s;
    a.output_stride_s = p->output_stride_s;
    a.cache_stride_s = p->cache_stride_s;
    a.cache_stride_l = p->cache_stride_l;
    a.cache_stride_h = p->cache_stride_h;
    a.cache_stride_kv = p->cache_stride_kv;
    a.cachestarts_stride_b = p->cachestarts_stride_b;
    return launch_result("prefill_attention", pmxhip::launch_prefill(a, stream));
}

static int reorder_common(const char* what, bool invert, pmxhip_stream_t stream, const void* cache, const void* scale,
                          const void* outer, const int64_t* page_ids, const pmxhip_reorder_stride* src,
                          const pmxhip_reorder_stride* dst, int64_t page_nums, int64_t layers, int64_t kv_heads,
                          int64_t tokens, int64_t head_dim, int64_t group_size, int64_t tp_rank, int64_t tp_size)
{
    if (!src || !dst) return fail(PMXHIP_INVALID_VALUE, "%s: null stride", what);
    if (page_nums < 0 || layers < 0 || kv_heads < 0 || tokens < 0)
        return fail(PMXHIP_INVALID_VALUE, "%s: negative extent", what);
    if (page_nums == 0 || layers == 0 || kv_heads == 0 || tokens == 0) return PMXHIP_SUCCESS;
    if (!cache || !scale || !outer || !page_ids) return fail(PMXHIP_INVALID_VALUE, "%s: null device pointer", what);
    if (head_dim <= 0 || group_size <= 0 || head_dim % group_size != 0)
        return fail(PMXHIP_INVALID_VALUE, "%s: head_dim must be a positive multiple of group_size", what);
    if (tp_size <= 0 || tp_rank < 0 || tp_rank >= tp_size) return fail(PMXHIP_INVALID_VALUE, "%s: tp_rank outside [0, tp_size)", what);
    const int64_t pcb = src->p_stride_cache, psb = src->p_stride_scale; // both directions read them from src_stride
    const int64_t slot = (pcb + psb) * tp_size;
    const int64_t scale_row = head_dim / group_size * 2;
    // cache side / outer side strides of each direction
    const pmxhip_reorder_stride* cs = invert ? dst : src; // cache-side strides
    const pmxhip_reorder_stride* os = invert ? src : dst; // outer-side strides
    for (int part = 0; part < 2; ++part) {
        pmxhip::PageCopyLaunch a{};
        a.page_ids = page_ids;
        a.pages = page_nums;
        a.layers = layers;
        a.kv_heads = kv_heads;
        a.tokens = tokens;
        a.row_bytes = part == 0 ? head_dim : scale_row;
        const int64_t c_stride[5] = {part == 0 ? cs->l_stride_cache : cs->l_stride_scale, part == 0 ? cs->kv_stride_cache : cs->kv_stride_scale,
                                     part == 0 ? cs->h_stride_cache : cs->h_stride_scale, part == 0 ? cs->t_stride_cache : cs->t_stride_scale,
                                     part == 0 ? cs->d_stride_cache : cs->d_stride_scale};
        const int64_t o_stride[5] = {part == 0 ? os->l_stride_cache : os->l_stride_scale, part == 0 ? os->kv_stride_cache : os->kv_stride_scale,
                                     part == 0 ? os->h_stride_cache : os->h_stride_scale, part == 0 ? os->t_stride_cache : os->t_stride_scale,
                                     part == 0 ? os->d_stride_cache : os->d_stride_scale};
        const char* c_base = static_cast<const char*>(part == 0 ? cache : scale);
        const char* o_base = static_cast<const char*>(outer) + tp_rank * pcb + (part == 0 ? 0 : (tp_size - tp_rank) * pcb + tp_rank * psb);
        const int64_t c_page = head_dim * a.row_bytes; // kv_cache_reorder.cu:44, 57
        for (int i = 0; i < 5; ++i) {
            a.src_stride[i] = invert ? o_stride[i] : c_stride[i];
            a.dst_stride[i] = invert ? c_stride[i] : o_stride[i];
        }
        a.src = invert ? o_base : c_base;
        a.dst = const_cast<char*>(invert ? c_base : o_base);
        a.src_slot_stride = invert ? slot : 0;
        a.dst_slot_stride = invert ? 0 : slot;
        a.src_page_stride = invert ? 0 : c_page;
        a.dst_page_stride = invert ? c_page : 0;
        pmxhip::launch_page_copy(a, stream);
    }
    return launch_status(what);
}

int pmxhip_kv_cache_reorder(pmxhip_stream_t stream, const void* kv_cache, const void* kv_scale, const int64_t* page_ids,
                            const pmxhip_reorder_stride* src_stride, const pmxhip_reorder_stride* dst_stride, int64_t page_nums,
                            int64_t layers, int64_t kv_heads, int64_t tokens, int64_t head_dim, int64_t group_size,
                            int64_t tp_rank, int64_t tp_size, void* outer_mem)
{
    return reorder_common("kv_cache_reorder", false, stream, kv_cache, kv_scale, outer_mem, page_ids, src_stride, dst_stride,
                          page_nums, layers, kv_heads, tokens, head_dim, group_size, tp_rank, tp_size);
}

int pmxhip_kv_cache_invert_reorder(pmxhip_stream_t stream, const void* outer_mem, const int64_t* page_ids,
                                   const pmxhip_reorder_stride* src_stride, const pmxhip_reorder_stride* dst_stride,
                                   int64_t page_nums, int64_t layers, int64_t kv_heads, int64_t tokens, int64_t head_dim,
                                   int64_t group_size, int64_t tp_rank, int64_t tp_size, void* kv_cache, void* kv_scale)
{
    return reorder_common("kv_cache_invert_reorder", true, stream, kv_cache, kv_scale, outer_mem, page_ids, src_stride, dst_stride,
                          page_nums, layers, kv_heads, tokens, head_dim, group_size, tp_rank, tp_size);
}

static int rope_common(const char* what, const pmxhip_rope_params* p, const pmxhip_kvstore_params* st, pmxhip_stream_t stream)
{
    if (!p) return fail(PMXHIP_INVALID_VALUE, "%s: null params", what);
    if (p->head_dim <= 0 || p->head_dim % 8 != 0 || p->head_dim > 256)
        return fail(PMXHIP_UNSUPPORTED, "%s: head_dim must be a multiple of 8, at most 256", what);
    if (p->rotary_dim < 0 || p->rotary_dim % 2 != 0 || p->rotary_dim > p->head_dim) // rotary_position_embedding.cu:395-398
        return fail(PMXHIP_INVALID_VALUE, "%s: rotary_dim should be an even number not above head_dim", what);
    if (p->scaling_type < 0 || p->scaling_type > 2) return fail(PMXHIP_INVALID_VALUE, "%s: invalid scaling type: %d", what, p->scaling_type);
    if (p->scaling_type != 0 && !(p->scaling_factor > 0.f)) return fail(PMXHIP_INVALID_VALUE, "%s: scaling_factor must be positive", what);
    if (p->batch < 0 || p->max_seqlen < 0 || p->num_heads <= 0 || p->num_key_heads < 0 || p->num_key_heads > p->num_heads)
        return fail(PMXHIP_INVALID_VALUE, "%s: bad batch/max_seqlen/heads", what);
    if (p->batch == 0 || p->max_seqlen == 0) return PMXHIP_SUCCESS;
    if (!p->query || !p->key || !p->start_pos || !p->seqstarts || !p->rotated_query || (!st && !p->rotated_key))
        return fail(PMXHIP_INVALID_VALUE, "%s: null device pointer", what);
    if (!aligned16(p->query) || !aligned16(p->key) || !aligned16(p->rotated_query) || (p->rotated_key && !aligned16(p->rotated_key)) ||
        p->query_stride_s % 8 || p->key_stride_s % 8 || p->rotated_query_stride_s % 8 || p->rotated_key_stride_s % 8)
        return fail(PMXHIP_UNSUPPORTED, "%s: rows must be 16-byte aligned", what);

    pmxhip::RopeLaunch a{};
    a.query = p->query;
    a.key = p->key;
    a.rotated_query = p->rotated_query;
    a.rotated_key = p->rotated_key;
    a.seqstarts = p->seqstarts;
    a.start_pos = p->start_pos;
    a.batch = p->batch;
    a.max_tokens = p->batch * p->max_seqlen;
    a.num_heads = p->num_heads;
    a.num_key_heads = p->num_key_heads;
    a.head_dim = (int32_t)p->head_dim;
    a.rotary_dim = (int32_t)p->rotary_dim;
    a.query_stride_s = p->query_stride_s;
    a.key_stride_s = p->key_stride_s;
    a.rotated_query_stride_s = p->rotated_query_stride_s;
    a.rotated_key_stride_s = p->rotated_key_stride_s;
    a.theta = p->theta;
    a.scaling_factor = p->scaling_factor;
    a.max_position_embeddings = p->max_position_embeddings;
    a.scaling_type = p->scaling_type;
    a.bypass_key = p->bypass_key;
    if (st) {
        if (st->head_dim != p->head_dim || st->num_kv_heads != p->num_key_heads || st->batch != p->batch ||
            st->seqstarts != p->seqstarts || st->start_pos != p->start_pos)
            return fail(PMXHIP_INVALID_VALUE, "%s: the append part must describe the same rows as the rotation", what);
        if (int rc = check_cache_layout(what, st->cache_mode, st->page_size, st->cache_stride_s, st->cache_stride_l,
                                        st->cache_stride_h, st->cache_stride_kv, 8))
            return rc;
        if (!st->current_value || !st->cachestarts || !st->cache || !st->scale)
            return fail(PMXHIP_INVALID_VALUE, "%s: null device pointer", what);
        if (st->current_value_stride_s % 8 || !aligned16(st->current_value) || (reinterpret_cast<uintptr_t>(st->cache) & 7u))
            return fail(PMXHIP_UNSUPPORTED, "%s: current_value needs 16-byte aligned rows, cache 8-byte alignment", what);
        a.value = st->current_value;
        a.value_stride_s = st->current_value_stride_s;
        a.cache = static_cast<int8_t*>(st->cache);
        a.scale = st->scale;
        a.cachestarts = st->cachestarts;
        a.layer_idx = st->layer_idx;
        a.cache_stride_s = st->cache_stride_s;
        a.cache_stride_l = st->cache_stride_l;
        a.cache_stride_h = st->cache_stride_h;
        a.cache_stride_kv = st->cache_stride_kv;
        a.cachestarts_stride_b = st->cachestarts_stride_b;
        a.cache_mode = st->cache_mode;
    }
    return launch_result(what, pmxhip::launch_rope(a, current_compute_units(), stream));
}

int pmxhip_rotary_position_embedding(const pmxhip_rope_params* p, pmxhip_stream_t stream)
{
    return rope_common("rotary_position_embedding", p, nullptr, stream);
}

int pmxhip_rope_kv_cache_quantize(const pmxhip_rope_params* rope, const pmxhip_kvstore_params* store, pmxhip_stream_t stream)
{
    if (!store) return fail(PMXHIP_INVALID_VALUE, "rope_kv_cache_quantize: null params");
    return rope_common("rope_kv_cache_quantize", rope, store, stream);
}

int64_t pmxhip_row_parallel_linear_workspace_size(int64_t m, int64_t in_features, int64_t out_features)
{
    return pmxhip_row_parallel_linear_workspace_size_ex(m, in_features, out_features, 0);
}

int64_t pmxhip_row_parallel_linear_workspace_size_ex(int64_t m, int64_t in_features, int64_t out_features, int32_t flags)
{
    if (m <= 0 || in_features <= 0 || out_features <= 0) return 0;
    const int64_t own = pmxhip::linear_workspace_bytes(m, out_features, in_features, current_compute_units());
    if ((flags & PMXHIP_LINEAR_VENDOR_GEMM) && m >= pmxhip::kLinearLibraryRows && pmxhip::linear_library_available() &&
        own < pmxhip::kLinearLibraryWorkspace)
        return pmxhip::kLinearLibraryWorkspace;
    return own;
}

int pmxhip_row_parallel_linear(pmxhip_stream_t stream, const void* input, const void* weight, const void* bias, int64_t m,
                               int64_t in_features, int64_t out_features, int64_t input_stride, int64_t weight_stride,
                               int64_t output_stride, int64_t workspace_size, void* workspace, void* output)
{
    return pmxhip_row_parallel_linear_ex(stream, input, weight, bias, m, in_features, out_features, input_stride, weight_stride,
                                         output_stride, workspace_size, workspace, output, 0);
}

int pmxhip_row_parallel_linear_ex(pmxhip_stream_t stream, const void* input, const void* weight, const void* bias, int64_t m,
                                  int64_t in_features, int64_t out_features, int64_t input_stride, int64_t weight_stride,
                                  int64_t output_stride, int64_t workspace_size, void* workspace, void* output, int32_t flags)
{
    if (flags & ~PMXHIP_LINEAR_VENDOR_GEMM) return fail(PMXHIP_INVALID_VALUE, "row_parallel_linear: unknown flags %d", flags);
    if (m < 0 || in_features <= 0 || out_features <= 0) return fail(PMXHIP_INVALID_VALUE, "row_parallel_linear: bad sizes");
    if (m == 0) return PMXHIP_SUCCESS;
    if (!input || !weight || !output) return fail(PMXHIP_INVALID_VALUE, "row_parallel_linear: null device pointer");
    if (out_features % 16 != 0 || in_features % 32 != 0)
        return fail(PMXHIP_UNSUPPORTED, "row_parallel_linear: out_features must be a multiple of 16 and in_features of 32 "
                                        "(got %lld, %lld)", (long long)out_features, (long long)in_features);
    if (input_stride < in_features || weight_stride < in_features || output_stride < out_features)
        return fail(PMXHIP_INVALID_VALUE, "row_parallel_linear: a row stride is shorter than its row");
    if (!aligned16(input) || !aligned16(weight) || input_stride % 8 != 0 || weight_stride % 8 != 0 ||
        (reinterpret_cast<uintptr_t>(output) & 7u) || output_stride % 4 != 0 || (bias && (reinterpret_cast<uintptr_t>(bias) & 7u)))
        return fail(PMXHIP_UNSUPPORTED, "row_parallel_linear: input and weight rows must be 16-byte aligned, output rows and bias 8-byte aligned");
    pmxhip::LinearLaunch a{};
    a.input = input;
    a.weight = weight;
    a.bias = bias;
    a.output = output;
    a.m = m;
    a.n = out_features;
    a.k = in_features;
    a.input_stride = input_stride;
    a.weight_stride = weight_stride;
    a.output_stride = output_stride;
    // on request, many rows: a compute-bound GEMM for the vendor library, when it can be loaded and takes the problem
    if ((flags & PMXHIP_LINEAR_VENDOR_GEMM) && m >= pmxhip::kLinearLibraryRows && pmxhip::linear_library_available()) {
        int device = 0;
        if (hipGetDevice(&device) != hipSuccess) return fail(PMXHIP_OTHER_ERROR, "row_parallel_linear: no current device");
        const int rc = pmxhip::launch_linear_library(a, device, workspace, workspace ? workspace_size : 0, stream);
        if (rc != pmxhip::kLaunchNoKernel) return launch_result("row_parallel_linear", rc);
    }
    return launch_result("row_parallel_linear",
                         pmxhip::launch_linear(a, current_compute_units(), workspace, workspace ? workspace_size : 0, stream));
}

} // extern "C"
