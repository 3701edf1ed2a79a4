// Kernel argument blocks and launcher prototypes shared between the host layer
// (c_api.cpp) and the .hip translation units.
#ifndef PMX_HIP_LAUNCH_PARAMS_H_
#define PMX_HIP_LAUNCH_PARAMS_H_

#include <hip/hip_runtime_api.h>
#include <stdint.h>

#include <atomic>

namespace pmxhip {

struct QuantLaunch {
    const void* current_key;
    const void* current_value;
    const int64_t* seqstarts;
    const int64_t* cachestarts;
    const int64_t* start_pos;
    int8_t* cache;
    void* scale;
    int64_t batch;
    int64_t layer_idx;
    int32_t num_kv_heads;
    int32_t head_dim;
    int64_t current_key_stride_s;
    int64_t current_value_stride_s;
    int64_t cache_stride_s;
    int64_t cache_stride_l;
    int64_t cache_stride_h;
    int64_t cache_stride_kv;
    int64_t cachestarts_stride_b;
    int64_t max_tokens; // batch * max_seqlen: upper bound of the new-token count
    int32_t cache_mode;
};

struct DecodeLaunch {
    const void* query;
    const void* attn_mask;
    void* output;
    const void* cache;
    const void* scale;
    const int64_t* cachestarts;
    const int64_t* kvstarts;
    float* partial_out; // (ranges + batches, Hq, D)
    float* partial_ml;  // (ranges + batches, Hq, 2)
    float attn_scale;
    int32_t cache_mode;
    int64_t layer_idx;
    int64_t num_kv_repeats;
    int64_t query_stride_s;
    int64_t output_stride_s;
    int64_t mask_stride_s;
    int64_t mask_stride_h;
    int64_t cache_stride_s;
    int64_t cache_stride_l;
    int64_t cache_stride_h;
    int64_t cache_stride_kv;
    int64_t cachestarts_stride_b;
    int64_t decoding_batches;
    int64_t num_heads;
    int64_t num_kv_heads;
    int32_t head_dim;
    int32_t ranges;               // workgroups along the kv-token stream
    int32_t kv_heads_per_group;   // kv heads per workgroup (power of two)
    int32_t q_heads_per_pass;     // GT
    int32_t num_passes;           // ceil(num_kv_repeats / GT)
    int32_t wg_tokens;            // tokens one workgroup iteration covers: the unit of the range cuts, a property
                                  // of the kernel named by `kernel` (the combine kernel derives the same cuts from it)
    int32_t min_tokens_per_range;
    int32_t kernel;               // DecodeKernel that runs the token ranges; never kDecodeKernelAuto at launch
    // Chunks of a few query tokens per sequence on the 32-column kernel (nullptr = one query token per sequence, row =
    // sequence index): rows of sequence b are seqstarts[b] .. seqstarts[b + 1]; num_kv_repeats and num_heads then count
    // (query position, query head) columns, chunk_q_heads the query heads per kv head.
    const int64_t* seqstarts;
    int32_t chunk_q_heads;
    int32_t chunk_causal;
};

struct PrefillLaunch {
    const void* query;
    void* output;
    const void* cache;
    const void* scale;
    const int64_t* seqstarts;   // already offset to the first prefill sequence
    const int64_t* kvstarts;    // likewise
    const int64_t* cachestarts; // likewise
    float attn_scale;
    int32_t is_causal;
    int32_t cache_mode;
    int64_t prefill_batches;
    int64_t max_seqlen;
    int64_t query_rows;         // rows of the prefill sequences, 0 = unknown (bounds the launch only)
    int64_t layer_idx;
    int64_t num_heads;
    int64_t num_kv_heads;
    int32_t head_dim;
    int64_t query_stride_s;
    int64_t output_stride_s;
    int64_t cache_stride_s;
    int64_t cache_stride_l;
    int64_t cache_stride_h;
    int64_t cache_stride_kv;
    int64_t cachestarts_stride_b;
    // optional inputs
    const void* attn_mask;      // half, additive; NULL = none
    int64_t mask_stride_s;
    int64_t mask_stride_h;
    const float* alibi_slopes;  // float32 per query head; NULL = none
    // K/V from the step's own fp16 rows instead of the cache (kv length = query length; kvstarts = seqstarts)
    const void* current_key;    // NULL = attend over the cache
    const void* current_value;
    int64_t key_stride_s;
    int64_t value_stride_s;
};

// One strided copy of whole pages (cache bytes or scale bytes) between the cache and the outer buffer.
struct PageCopyLaunch {
    const char* src;
    char* dst;
    const int64_t* page_ids;
    int64_t pages, layers, kv_heads, tokens, row_bytes;
    int64_t src_slot_stride, dst_slot_stride; // per slot (index into page_ids)
    int64_t src_page_stride, dst_page_stride; // per page id
    int64_t src_stride[5], dst_stride[5];     // layer, K/V plane, kv head, token, byte
};

// Rotary position embedding of the step's Q and K rows, optionally fused with the quantise/append of
// the rotated K and of V (cache != nullptr).
struct RopeLaunch {
    const void* query;          // half (S, Hq, D)
    const void* key;            // half (S, KVH, D)
    const void* value;          // half (S, KVH, D); only read when appending
    void* rotated_query;        // half; may alias query
    void* rotated_key;          // half; may be nullptr when appending
    const int64_t* seqstarts;   // (B + 1)
    const int64_t* start_pos;   // (B)
    int64_t batch;
    int64_t max_tokens;         // upper bound of the number of rows
    int64_t num_heads, num_key_heads;
    int32_t head_dim, rotary_dim;
    int64_t query_stride_s, key_stride_s, value_stride_s, rotated_query_stride_s, rotated_key_stride_s; // in halves
    float theta, scaling_factor;
    int64_t max_position_embeddings;
    int32_t scaling_type;       // 0 none, 1 linear, 2 dynamic
    int32_t bypass_key;
    // 1 / theta^(i / (rotary_dim / 2)) for pair i, computed by the host launcher (in double, rounded to float) when
    // theta does not depend on the sequence (scaling types 0 and 1); has_inv_freq = 0: the kernel computes it
    float inv_freq[128];
    int32_t has_inv_freq;
    int32_t tokens_per_wg;      // consecutive tokens one workgroup takes, at most 256 / (head_dim / 2)
    // append part (same meaning as QuantLaunch)
    int8_t* cache;
    void* scale;
    const int64_t* cachestarts;
    int64_t layer_idx;
    int64_t cache_stride_s, cache_stride_l, cache_stride_h, cache_stride_kv, cachestarts_stride_b;
    int32_t cache_mode;
};

// Return codes of the launchers below.
constexpr int kLaunchOk = 0;
constexpr int kLaunchNoKernel = 1;      // no kernel serves the shape
constexpr int kLaunchNeedsWarmup = 2;   // the kernel's one-time attribute call is due, but the stream is being captured

// output(M, N) = input(M, K) * weight(N, K)^T + bias; half everywhere, strides in halves per row
struct LinearLaunch {
    const void* input;
    const void* weight;
    const void* bias;   // half (N) or nullptr
    void* output;
    int64_t m, n, k;
    int64_t input_stride, weight_stride, output_stride;
};
// workspace: float32 partial tiles of the k ranges (linear_workspace_bytes; may be null: then one k range)
int launch_linear(const LinearLaunch& a, int compute_units, void* workspace, int64_t workspace_bytes, hipStream_t stream);
int64_t linear_workspace_bytes(int64_t m, int64_t n, int64_t k, int compute_units);

// The one-time hipFuncSetAttribute of a kernel whose dynamic LDS exceeds the default limit: once per kernel and
// device (`ready` holds a bit per device; devices 0-63, like the other per-device caches of the library -- a
// device beyond them is refused, not aliased).  It runs before the kernel's first launch on the device and never
// while `stream` is being captured into a graph: a caller that captures first gets kLaunchNeedsWarmup and calls
// pmxhip_init() or one eager step before.
using DeviceMask = std::atomic<uint64_t>;
inline uint64_t current_device_bit()
{
    int device = 0;
    if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= 64) return 0;
    return uint64_t(1) << device;
}
inline int set_dynamic_lds_once(const void* kernel, int bytes, DeviceMask& ready)
{
    const uint64_t bit = current_device_bit();
    if (bit == 0) return kLaunchNoKernel;
    if (ready.load(std::memory_order_acquire) & bit) return kLaunchOk;
    if (hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes) != hipSuccess) return kLaunchNoKernel;
    ready.fetch_or(bit, std::memory_order_release);
    return kLaunchOk;
}
inline int ensure_dynamic_lds(const void* kernel, int bytes, hipStream_t stream, DeviceMask& ready)
{
    const uint64_t bit = current_device_bit();
    if (bit != 0 && (ready.load(std::memory_order_acquire) & bit)) return kLaunchOk;
    hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &st) != hipSuccess || st != hipStreamCaptureStatusNone) {
        (void)hipGetLastError();
        return kLaunchNeedsWarmup;
    }
    return set_dynamic_lds_once(kernel, bytes, ready);
}

// Rows from which the output projection is a compute-bound GEMM and, when the caller asks for it
// (PMXHIP_LINEAR_VENDOR_GEMM), goes to the vendor library where that can be loaded (linear_library.cpp); up to here
// this build's weight-streaming kernels are as fast or faster.
constexpr int64_t kLinearLibraryRows = 384;
constexpr int64_t kLinearLibraryWorkspace = 64 << 20; // what the library is offered when the caller asks how much to bring
bool linear_library_available();
int init_linear_library(int device);
int launch_linear_library(const LinearLaunch& a, int device, void* workspace, int64_t workspace_bytes, hipStream_t stream);
int launch_kv_quantize(const QuantLaunch& a, int compute_units, hipStream_t stream);
int launch_rope(const RopeLaunch& a, int compute_units, hipStream_t stream);
void launch_page_copy(const PageCopyLaunch& a, hipStream_t stream);
int launch_decode(const DecodeLaunch& a, int stage, hipStream_t stream); // stage: 0 both, 1 ranges, 2 combine

// ---- which kernel runs the token ranges of a decode step (decode_select.cpp; host only) ----
// The values are those of pmxhip_decode_kernel_t in the C header.
enum DecodeKernel : int32_t {
    kDecodeKernelAuto = 0,    // as a request: by shape
    kDecodeKernelGeneral = 1, // decode_attn.hip: VALU, every head_dim and head count, up to 8 query heads per pass
    kDecodeKernelQuad = 2,    // decode_attn_quad.hip: 4x4x4 MFMA per quad; head_dim 64 or 128 (two or more kv heads) or 256
    kDecodeKernelMfma16 = 3,  // decode_attn_mfma.hip: 16 query-head columns, head_dim 128
    kDecodeKernelMfma32 = 4,  // decode_attn_mfma.hip: 32 query-head columns per pass, head_dim 128 or 64
};
// Fewest tokens a range is given: with fewer, the start of a piece (lookups, query rows, first rows of the cache) and
// its slot in the workspace cost more than the parallelism buys.  On batches far smaller than the chip 64 beats 128
// (one sequence of 4096 tokens: 12.7 against 18.1 us for the kernel; 32 sequences of 200-600 tokens: 22.1 against
// 26.4 us per layer call) and 32 is slower again; where ranges of 128 already fill half of the workgroup slots they
// are the better cut (one sequence of 32768 tokens: 21.9 against 24.5 us), which is how the plan chooses its number
// of ranges.  Batches that fill the chip are cut by the number of workgroup slots, not by this.
constexpr int decode_min_tokens_per_range(int wg_tokens) { return wg_tokens > 64 ? wg_tokens : 64; }
// ... and the floor that the kernels apply to whatever number of ranges they are given: a step of a few sequences
// that leaves most CUs without a workgroup is cut down to this (one sequence of 4096 tokens: 12.7 us for the kernel
// with 64 ranges of 64 tokens, 10.2 us with 128 of 32).
constexpr int decode_floor_tokens_per_range(int wg_tokens) { return wg_tokens > 32 ? wg_tokens : 32; }

struct DecodeChoice {
    int32_t kernel;             // never kDecodeKernelAuto
    int32_t kv_heads_per_group; // kv heads one workgroup serves
    int32_t q_heads_per_pass;   // query heads per kv head served by one pass (general kernel: 1, 2, 4 or 8)
    int32_t num_passes;
    int32_t wg_tokens;          // tokens per workgroup iteration = unit of the range cuts
    int32_t wgs_per_cu;         // workgroups per CU that a long stream is cut for (sizes the number of ranges)
    int32_t wgs_per_cu_short;   // ... and that a CU can hold: what short batches, whose ranges are a few blocks, are spread over
};
// The kernel that serves a shape, and the grouping it implies.  `requested` kDecodeKernelAuto picks by shape;
// any other value insists on that kernel and the call fails (false) when it cannot serve the shape.
bool decode_choose(int64_t head_dim, int64_t num_heads, int64_t num_kv_heads, int32_t requested, DecodeChoice* out);
// Makes the choice fit a cache layout: the kernels address a row as a 64-bit base per wave plus a 32-bit offset per
// lane, and where the kv heads of a wave lie further apart than such an offset reaches (cache_stride_h of a layout
// that keeps the heads outermost) the general kernel takes fewer kv heads per workgroup and, unless the quad kernel
// was requested, a kernel with a wave per kv head takes its steps.  The number of ranges of a plan stays valid: it
// does not depend on the grouping.  False: no kernel serves the strides (a block of tokens alone spans 2 GiB, or a
// stride is negative).
bool decode_fit_cache_strides(int64_t head_dim, int64_t num_heads, int64_t num_kv_heads, int32_t requested,
                              int64_t stride_s, int64_t stride_h, DecodeChoice* c);
// What the quad kernel needs of a launch beyond the C ABI's own checks: 16-byte aligned output rows and,
// with attn_mask, one set of waves and mask offsets within 32 bits.
bool decode_quad_launch_ok(const DecodeLaunch& a);
const char* decode_kernel_name(int32_t kernel);
int decode_wg_tokens(int head_dim, int kv_heads_per_group); // of the general kernel
constexpr int kDecodeQuadTokens = 16;
constexpr int kDecodeMfmaWavesPerCu = 8; // 20 KB of LDS per wave
constexpr int kDecodeMfmaTokens = 32;
constexpr int kDecodeMfma16Columns = 16;
constexpr int kDecodeMfmaColumns = 32;
void launch_decode_quad(const DecodeLaunch& a, hipStream_t stream);
void launch_decode_mfma(const DecodeLaunch& a, hipStream_t stream);
// One-time attribute calls of the kernels whose dynamic LDS exceeds the default limit, all variants at once.
int init_decode_kernels();
int init_prefill_kernels();
void launch_splitkv_combine_rows(const float* partial_out, const float* partial_ml, const int64_t* piece_begin,
                                 const int64_t* piece_end, int64_t rows, int64_t head_dim, void* output,
                                 hipStream_t stream);
int launch_prefill(const PrefillLaunch& a, hipStream_t stream);

} // namespace pmxhip

#endif // PMX_HIP_LAUNCH_PARAMS_H_
