// Kernel argument blocks and launcher prototypes shared between the host layer
// (c_api.cpp) and the .hip translation units.
#ifndef PMX_HIP_LAUNCH_PARAMS_H_
#define PMX_HIP_LAUNCH_PARAMS_H_

#include <hip/hip_runtime_api.h>
#include <stdint.h>

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
    int32_t wg_tokens;            // tokens one workgroup iteration covers
    int32_t min_tokens_per_range;
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
    // append part (same meaning as QuantLaunch)
    int8_t* cache;
    void* scale;
    const int64_t* cachestarts;
    int64_t layer_idx;
    int64_t cache_stride_s, cache_stride_l, cache_stride_h, cache_stride_kv, cachestarts_stride_b;
    int32_t cache_mode;
};

int launch_kv_quantize(const QuantLaunch& a, hipStream_t stream);
int launch_rope(const RopeLaunch& a, hipStream_t stream);
void launch_page_copy(const PageCopyLaunch& a, hipStream_t stream);
int launch_decode(const DecodeLaunch& a, int stage, hipStream_t stream); // stage: 0 both, 1 ranges, 2 combine
int decode_wg_tokens(int head_dim, int kv_heads_per_group);
bool decode_general_forced(); // PMX_HIP_DECODE_GENERAL=1 in the environment: every shape on the general kernel
bool decode_quad_shape(int64_t head_dim, int64_t num_heads, int64_t num_kv_heads); // head_dim 128 (even number of kv heads) or 256, <= 4 query heads each
int decode_quad_kv_heads(int64_t head_dim, int64_t num_kv_heads);                  // kv heads per workgroup: 8, 4 or 2 (head_dim 256: 4, 2 or 1)
bool decode_quad_mask_ok(int64_t num_heads, int64_t num_kv_repeats, int64_t mask_stride_h); // attn_mask within its reach
bool decode_quad_applicable(const DecodeLaunch& a);
constexpr int kDecodeQuadTokens = 16;
void launch_decode_quad(const DecodeLaunch& a, hipStream_t stream);
// head_dim 128, 5 to 32 query heads per kv head, kv heads in fours: MFMA kernel, groups of four kv heads, 32-token blocks
bool decode_mfma_shape(int64_t head_dim, int64_t num_heads, int64_t num_kv_heads);
bool decode_mfma_applicable(const DecodeLaunch& a);
void launch_decode_mfma(const DecodeLaunch& a, hipStream_t stream);
int decode_mfma_kv_heads(int64_t num_kv_heads); // kv heads (= waves) per workgroup: 4, 2 or 1
constexpr int kDecodeMfmaWavesPerCu = 8;         // 16 KB of LDS per wave
constexpr int kDecodeMfmaTokens = 32;
constexpr int kDecodeMfmaColumns = 32;
void launch_splitkv_combine_rows(const float* partial_out, const float* partial_ml, const int64_t* piece_begin,
                                 const int64_t* piece_end, int64_t rows, int64_t head_dim, void* output,
                                 hipStream_t stream);
int launch_prefill(const PrefillLaunch& a, hipStream_t stream);

} // namespace pmxhip

#endif // PMX_HIP_LAUNCH_PARAMS_H_
