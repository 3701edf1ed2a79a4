// Decode attention over the int8 group-8 KV cache for gfx950 (wave64), plus the
// split-KV combine kernel.
//
// Semantics follow the reference decode kernels
// (src/ppl/kernel/llm/cuda/pmx/multi_head_cache_attention/kernel.cu:229-679 and
// 682-1057): one query token per sequence, kv head = q head / num_kv_repeats
// (kernel.cu:299), kv length = kvstarts[b+1]-kvstarts[b] (kernel.cu:347), token
// addressing of kernel.cu:365-368, logit = attn_scale * q.k (+ mask,
// kernel.cu:410-415), softmax, PV.  The decomposition is this file's own:
//
//   * The kv tokens of all decode sequences form one stream of T tokens.  It is
//     cut into `ranges` equal token ranges; workgroup x owns range x, whatever
//     sequences it covers ("pieces").  Ragged batches therefore load-balance by
//     construction.
//   * A workgroup serves KVHB kv heads at once and, per kv head, up to GT query
//     heads from registers, so every cache byte is fetched once per pass.
//   * A lane owns 16 consecutive channels of one (token, kv head): one 128-bit
//     load of int8 K, one of int8 V and one 32-bit load each for their two
//     scales.  LPS = D/16 lanes form a "slot" that walks tokens; a wave has
//     64/LPS slots, distributed over kv heads first and tokens second, so that a
//     wave's load instruction covers a contiguous run of the token row.
//   * Each slot keeps an online-softmax state per query head; slots are merged
//     through LDS at the end of a piece.  A piece that is a whole sequence is
//     written as final fp16 output; otherwise a float32 partial (normalised
//     output, running max, exp-sum) goes to the workspace and the combine kernel
//     merges the pieces of each sequence (kernel.cu:617-665 is the reference's
//     fused form of that merge).
#include "device_common.h"
#include "launch_params.h"

namespace pmxhip {

namespace {

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kNegBig = -1.0e30f; // finite "no token yet" running max (log2 units)
constexpr float kPShift = 14.0f;    // p = 2^(s - max + 14): keeps small p out of the fp16 subnormal range

constexpr int kDecodeThreads = 256;
constexpr int kDecodeWaves = kDecodeThreads / kWave;
constexpr int kTB = 8; // tokens a slot handles per block

struct RangeInfo {
    int64_t total;   // T
    int64_t per;     // tokens per range
};

// Tokens per range: equal shares rounded up to a whole number of workgroup
// iterations, never below kMinTokensPerRange.  Shared by both kernels.
__device__ __forceinline__ int64_t tokens_per_range(int64_t total, int ranges, int wg_tokens, int min_tokens)
{
    int64_t per = (total + ranges - 1) / ranges;
    if (per < min_tokens) per = min_tokens;
    return (per + wg_tokens - 1) / wg_tokens * wg_tokens;
}

// first b in [0, n) with starts[b + 1] - starts[0] > g   (starts is non-decreasing)
__device__ __forceinline__ int find_sequence(const int64_t* __restrict__ starts, int n, int64_t g)
{
    const int64_t base = starts[0];
    int lo = 0, hi = n; // answer in [lo, hi]
    while (lo < hi) {
        const int mid = (lo + hi) >> 1;
        if (starts[mid + 1] - base > g) hi = mid;
        else lo = mid + 1;
    }
    return lo;
}

} // namespace

// D: head dim (64, 96, 128, 256).  GT: query heads per kv head held in registers.
template <int D, int GT, bool PAGED, bool MASK>
__global__ __launch_bounds__(kDecodeThreads) void decode_attention_kernel(const DecodeLaunch a)
{
    constexpr int LPS = (D == 64) ? 4 : (D == 256 ? 16 : 8); // lanes per slot
    constexpr int LPS_ACTIVE = D / 16;                        // 6 of 8 for D = 96
    constexpr int SPW = kWave / LPS;                          // slots per wave
    constexpr int NSLOT = SPW * kDecodeWaves;

    __shared__ float sm_acc[NSLOT * D];
    __shared__ float sm_m[NSLOT];
    __shared__ float sm_l[NSLOT];

    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int ls = lane % LPS;            // lane in slot -> channels [16*ls, 16*ls+16)
    const int slot = lane / LPS;          // slot in wave
    const bool lane_on = ls < LPS_ACTIVE;
    const int ch0 = (lane_on ? ls : 0) * 16;

    // slots over (kv head, token sub-index): kv heads first
    const int kvhb = a.kv_heads_per_group;        // power of two, <= SPW
    const int tpl = SPW / kvhb;                   // tokens one wave load covers
    const int head_local = slot & (kvhb - 1);
    const int tsub = slot / kvhb;
    const int wave_tokens = kTB * tpl;            // tokens a wave handles per iteration
    const int wg_tokens = wave_tokens * kDecodeWaves;

    const int kvh = blockIdx.y * kvhb + head_local;
    const int g_first = blockIdx.z * GT; // first query head (within the kv head's group) of this pass
    const int G = (int)a.num_kv_repeats;

    const int64_t kv_base = a.kvstarts[0];
    const int64_t total = a.kvstarts[a.decoding_batches] - kv_base;
    const int64_t per = tokens_per_range(total, a.ranges, wg_tokens, a.min_tokens_per_range);
    const int64_t r0 = (int64_t)blockIdx.x * per;
    if (r0 >= total) return;
    const int64_t r1 = (r0 + per < total) ? r0 + per : total;

    const int8_t* __restrict__ cache = (const int8_t*)a.cache;
    const half_t* __restrict__ scale = (const half_t*)a.scale;
    const int64_t head_off = a.layer_idx * a.cache_stride_l + (int64_t)kvh * a.cache_stride_h + ch0;
    const float logit_scale = a.attn_scale * kLog2e;

    int b = find_sequence(a.kvstarts, (int)a.decoding_batches, r0);
    for (; b < a.decoding_batches; ++b) {
        const int64_t s_beg = a.kvstarts[b] - kv_base;
        if (s_beg >= r1) break;
        const int64_t s_end = a.kvstarts[b + 1] - kv_base;
        const int64_t len = s_end - s_beg;
        // piece [pa, pe) in sequence coordinates
        const int64_t pa = (r0 > s_beg ? r0 : s_beg) - s_beg;
        const int64_t pe = (r1 < s_end ? r1 : s_end) - s_beg;
        if (pe <= pa) continue;

        // ---- query heads of this kv head into registers (packed halves) ----
        half2_t q[GT][8];
#pragma unroll
        for (int g = 0; g < GT; ++g) {
            const int gi = g_first + g;
            const bool on = lane_on && gi < G;
            const int h = kvh * G + (gi < G ? gi : 0);
            const u32x4* qp = (const u32x4*)((const half_t*)a.query + (int64_t)b * a.query_stride_s + (int64_t)h * D + ch0);
            u32x4 lo = qp[0], hi = qp[1];
            if (!on) { lo = u32x4{0, 0, 0, 0}; hi = lo; }
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                q[g][i] = bitcast<half2_t>(lo[i]);
                q[g][4 + i] = bitcast<half2_t>(hi[i]);
            }
        }

        float m_run[GT], l_run[GT], acc[GT][16];
#pragma unroll
        for (int g = 0; g < GT; ++g) {
            m_run[g] = kNegBig;
            l_run[g] = 0.f;
#pragma unroll
            for (int c = 0; c < 16; ++c) acc[g][c] = 0.f;
        }

        const int64_t table_base = PAGED ? (int64_t)b * a.cachestarts_stride_b : (int64_t)b;
        const int64_t seq_row0 = PAGED ? 0 : a.cachestarts[b];
        const half_t* mask_row = nullptr;
        if (MASK) mask_row = (const half_t*)a.attn_mask + (int64_t)b * a.mask_stride_s + a.kvstarts[b];

        // iterations are aligned to wg_tokens in sequence coordinates so that a
        // wave's block never straddles a page
        for (int64_t it0 = pa / wg_tokens * wg_tokens; it0 < pe; it0 += wg_tokens) {
            const int64_t wave0 = it0 + (int64_t)wave * wave_tokens;
            if (wave0 >= pe || wave0 + wave_tokens <= pa) continue; // wave-uniform
            int64_t row_base;
            if (PAGED) {
                row_base = a.cachestarts[table_base + (wave0 >> 7)] + (wave0 & (kPage - 1));
            } else {
                row_base = seq_row0 + wave0;
            }

            u32x4 kq[kTB], vq[kTB];
            uint32_t ks[kTB], vs[kTB];
            bool valid[kTB];
#pragma unroll
            for (int j = 0; j < kTB; ++j) {
                const int tin = j * tpl + tsub; // token within the wave block
                const int64_t t = wave0 + tin;
                valid[j] = (t >= pa) && (t < pe);
                // clamp invalid tokens onto a valid one of this piece: the load is harmless, the logit is masked
                int64_t tc = t < pa ? pa : (t >= pe ? pe - 1 : t);
                const int64_t row = row_base + (tc - wave0);
                const int64_t off = row * a.cache_stride_s + head_off;
                kq[j] = *(const u32x4*)(cache + off);
                vq[j] = *(const u32x4*)(cache + off + a.cache_stride_kv);
                ks[j] = *(const uint32_t*)(scale + (off >> 3));
                vs[j] = *(const uint32_t*)(scale + ((off + a.cache_stride_kv) >> 3));
            }

            // ---- logits: s[g][j] in log2 units ----
            float s[GT][kTB];
#pragma unroll
            for (int j = 0; j < kTB; ++j) {
                half2_t kh[8];
#pragma unroll
                for (int w = 0; w < 4; ++w) {
                    const uint32_t f = kq[j][w] ^ kFlipSigns;
                    kh[2 * w] = cvt_bytes01(f);
                    kh[2 * w + 1] = cvt_bytes23(f);
                }
                const half2_t sc = bitcast<half2_t>(ks[j]);
                const float s0 = (float)sc.x * logit_scale;
                const float s1 = (float)sc.y * logit_scale;
#pragma unroll
                for (int g = 0; g < GT; ++g) {
                    float d0 = 0.f, d1 = 0.f;
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        d0 = dot2(q[g][i], kh[i], d0);
                        d1 = dot2(q[g][4 + i], kh[4 + i], d1);
                    }
                    float part = d0 * s0 + d1 * s1;
                    part = group_sum<LPS>(part);
                    if (MASK) {
                        const int h = kvh * G + g_first + g;
                        if (g_first + g < G && valid[j]) {
                            const int64_t t = wave0 + j * tpl + tsub;
                            part += (float)mask_row[(int64_t)h * a.mask_stride_h + t] * kLog2e;
                        }
                    }
                    s[g][j] = valid[j] ? part : -INFINITY;
                }
            }

            // ---- online softmax update, probabilities packed as halves ----
            half2_t p[GT][kTB / 2];
#pragma unroll
            for (int g = 0; g < GT; ++g) {
                float mx = s[g][0];
#pragma unroll
                for (int j = 1; j < kTB; ++j) mx = fmaxf(mx, s[g][j]);
                const float m_new = fmaxf(m_run[g], mx);
                const float alpha = __builtin_amdgcn_exp2f(m_run[g] - m_new);
                m_run[g] = m_new;
                const float bias = kPShift - m_new;
                float lsum = 0.f;
#pragma unroll
                for (int j = 0; j < kTB; j += 2) {
                    const float p0 = __builtin_amdgcn_exp2f(s[g][j] + bias);
                    const float p1 = __builtin_amdgcn_exp2f(s[g][j + 1] + bias);
                    const half2_t ph = bitcast<half2_t>(__builtin_amdgcn_cvt_pkrtz(p0, p1));
                    p[g][j / 2] = ph;
                    const half2_t ones = {(half_t)1.0f, (half_t)1.0f};
                    lsum = dot2(ph, ones, lsum); // the sum uses the rounded p, like the PV product
                }
                l_run[g] = l_run[g] * alpha + lsum;
#pragma unroll
                for (int c = 0; c < 16; ++c) acc[g][c] *= alpha;
            }

            // ---- PV: token pairs (j, j+1) share one dot2 per channel ----
#pragma unroll
            for (int j = 0; j < kTB; j += 2) {
                const u32x4 va = vq[j], vb = vq[j + 1];
                // scale pairs: (group0 of token j, group0 of token j+1), same for group1
                const half2_t sc0 = bitcast<half2_t>(__builtin_amdgcn_perm(vs[j + 1], vs[j], 0x05040100u));
                const half2_t sc1 = bitcast<half2_t>(__builtin_amdgcn_perm(vs[j + 1], vs[j], 0x07060302u));
                half2_t vh[16];
#pragma unroll
                for (int w = 0; w < 4; ++w) {
                    const half2_t sc = (w < 2) ? sc0 : sc1;
                    vh[4 * w + 0] = cvt_byte_pair<0>(va[w], vb[w]) * sc;
                    vh[4 * w + 1] = cvt_byte_pair<1>(va[w], vb[w]) * sc;
                    vh[4 * w + 2] = cvt_byte_pair<2>(va[w], vb[w]) * sc;
                    vh[4 * w + 3] = cvt_byte_pair<3>(va[w], vb[w]) * sc;
                }
#pragma unroll
                for (int g = 0; g < GT; ++g) {
#pragma unroll
                    for (int c = 0; c < 16; ++c) acc[g][c] = dot2(p[g][j / 2], vh[c], acc[g][c]);
                }
            }
        }

        // ---- merge the slots of each kv head through LDS, one query head at a time ----
        const bool whole = (pa == 0) && (pe == len);
        const int64_t piece = (int64_t)blockIdx.x + b;
        const int gslot = wave * SPW + slot;
        const int dup = NSLOT / kvhb; // slots per kv head
#pragma unroll
        for (int g = 0; g < GT; ++g) {
            __syncthreads();
            if (lane_on) {
#pragma unroll
                for (int c = 0; c < 16; c += 4) {
                    *(f32x4*)&sm_acc[gslot * D + ch0 + c] = f32x4{acc[g][c], acc[g][c + 1], acc[g][c + 2], acc[g][c + 3]};
                }
                if (ls == 0) {
                    sm_m[gslot] = m_run[g];
                    sm_l[gslot] = l_run[g];
                }
            }
            __syncthreads();
            const int gi = g_first + g;
            if (gi < G) {
                for (int idx = tid; idx < kvhb * D; idx += kDecodeThreads) {
                    const int hl = idx / D;
                    const int c = idx - hl * D;
                    // slots of kv head hl: every wave, slot index hl + kvhb * k
                    float M = kNegBig;
                    for (int k = 0; k < dup; ++k) {
                        const int sidx = (k / tpl) * SPW + hl + kvhb * (k % tpl);
                        M = fmaxf(M, sm_m[sidx]);
                    }
                    float L = 0.f, O = 0.f;
                    for (int k = 0; k < dup; ++k) {
                        const int sidx = (k / tpl) * SPW + hl + kvhb * (k % tpl);
                        const float w = __builtin_amdgcn_exp2f(sm_m[sidx] - M);
                        L += sm_l[sidx] * w;
                        O += sm_acc[sidx * D + c] * w;
                    }
                    const float o = L > 0.f ? O / L : 0.f;
                    const int h = (blockIdx.y * kvhb + hl) * G + gi;
                    if (whole) {
                        ((half_t*)a.output)[(int64_t)b * a.output_stride_s + (int64_t)h * D + c] = (half_t)o;
                    } else {
                        a.partial_out[(piece * a.num_heads + h) * D + c] = o;
                        if (c == 0) {
                            a.partial_ml[(piece * a.num_heads + h) * 2 + 0] = M;
                            a.partial_ml[(piece * a.num_heads + h) * 2 + 1] = L;
                        }
                    }
                }
            }
        }
        __syncthreads();
    }
}

// One workgroup per (sequence, query head): merges the pieces the decode kernel
// left in the workspace.  Sequences that fit one range were already written.
template <int D>
__global__ __launch_bounds__(64) void decode_combine_kernel(const DecodeLaunch a)
{
    const int b = blockIdx.y;
    const int h = blockIdx.x;
    const int lane = threadIdx.x;
    const int64_t kv_base = a.kvstarts[0];
    const int64_t total = a.kvstarts[a.decoding_batches] - kv_base;
    const int64_t s_beg = a.kvstarts[b] - kv_base;
    const int64_t s_end = a.kvstarts[b + 1] - kv_base;
    half_t* out = (half_t*)a.output + (int64_t)b * a.output_stride_s + (int64_t)h * D;
    if (s_end <= s_beg) { // empty sequence: the reference yields 0/(0+1e-6) = 0 (kernel.cu:516)
        for (int c = lane; c < D; c += 64) out[c] = (half_t)0.f;
        return;
    }
    const int64_t per = tokens_per_range(total, a.ranges, a.wg_tokens, a.min_tokens_per_range);
    const int64_t w0 = s_beg / per, w1 = (s_end - 1) / per;
    if (w0 == w1) return; // single piece, final output already written
    float M = kNegBig;
    for (int64_t w = w0; w <= w1; ++w) M = fmaxf(M, a.partial_ml[((w + b) * a.num_heads + h) * 2]);
    float o[(D + 63) / 64];
#pragma unroll
    for (int i = 0; i < (D + 63) / 64; ++i) o[i] = 0.f;
    float den = 0.f;
    for (int64_t w = w0; w <= w1; ++w) {
        const int64_t pi = (w + b) * a.num_heads + h;
        const float wt = a.partial_ml[pi * 2 + 1] * __builtin_amdgcn_exp2f(a.partial_ml[pi * 2] - M);
        den += wt;
#pragma unroll
        for (int i = 0; i < (D + 63) / 64; ++i) {
            const int c = lane + 64 * i;
            if (c < D) o[i] += wt * a.partial_out[pi * D + c];
        }
    }
    const float inv = den > 0.f ? 1.f / den : 0.f;
#pragma unroll
    for (int i = 0; i < (D + 63) / 64; ++i) {
        const int c = lane + 64 * i;
        if (c < D) out[c] = (half_t)(o[i] * inv);
    }
}

// Stand-alone merge over caller-supplied pieces (rows = (sequence, head) pairs).
__global__ __launch_bounds__(64) void splitkv_combine_rows_kernel(
    const float* __restrict__ partial_out, const float* __restrict__ partial_ml,
    const int64_t* __restrict__ piece_begin, const int64_t* __restrict__ piece_end,
    int64_t head_dim, half_t* __restrict__ output)
{
    const int64_t r = blockIdx.x;
    const int lane = threadIdx.x;
    const int64_t p0 = piece_begin[r], p1 = piece_end[r];
    float M = kNegBig;
    for (int64_t i = p0; i < p1; ++i)
        if (partial_ml[i * 2 + 1] > 0.f) M = fmaxf(M, partial_ml[i * 2]);
    for (int64_t c = lane; c < head_dim; c += 64) {
        float den = 0.f, o = 0.f;
        for (int64_t i = p0; i < p1; ++i) {
            const float l = partial_ml[i * 2 + 1];
            if (!(l > 0.f)) continue;
            const float wt = l * __builtin_amdgcn_exp2f(partial_ml[i * 2] - M);
            den += wt;
            o += wt * partial_out[i * head_dim + c];
        }
        output[r * head_dim + c] = (half_t)(den > 0.f ? o / den : 0.f);
    }
}

// ---- host-side launchers (called from the C ABI) -------------------------------

template <int D, int GT>
static void launch_decode_dgt(const DecodeLaunch& a, dim3 grid, hipStream_t stream)
{
    const bool paged = a.cache_mode == 1;
    const bool mask = a.attn_mask != nullptr;
    if (paged) {
        if (mask) hipLaunchKernelGGL((decode_attention_kernel<D, GT, true, true>), grid, dim3(kDecodeThreads), 0, stream, a);
        else hipLaunchKernelGGL((decode_attention_kernel<D, GT, true, false>), grid, dim3(kDecodeThreads), 0, stream, a);
    } else {
        if (mask) hipLaunchKernelGGL((decode_attention_kernel<D, GT, false, true>), grid, dim3(kDecodeThreads), 0, stream, a);
        else hipLaunchKernelGGL((decode_attention_kernel<D, GT, false, false>), grid, dim3(kDecodeThreads), 0, stream, a);
    }
}

template <int D>
static int launch_decode_d(const DecodeLaunch& a, int stage, hipStream_t stream)
{
    const dim3 grid((unsigned)a.ranges, (unsigned)(a.num_kv_heads / a.kv_heads_per_group), (unsigned)a.num_passes);
    if (stage != 2) {
        switch (a.q_heads_per_pass) {
            case 1: launch_decode_dgt<D, 1>(a, grid, stream); break;
            case 2: launch_decode_dgt<D, 2>(a, grid, stream); break;
            case 4: launch_decode_dgt<D, 4>(a, grid, stream); break;
            case 8: launch_decode_dgt<D, 8>(a, grid, stream); break;
            default: return 1;
        }
    }
    if (stage == 1) return 0;
    // always run: it also writes the zero rows of empty sequences
    hipLaunchKernelGGL((decode_combine_kernel<D>), dim3((unsigned)a.num_heads, (unsigned)a.decoding_batches), dim3(64), 0, stream, a);
    return 0;
}

int launch_decode(const DecodeLaunch& a, int stage, hipStream_t stream)
{
    switch (a.head_dim) {
        case 64: return launch_decode_d<64>(a, stage, stream);
        case 96: return launch_decode_d<96>(a, stage, stream);
        case 128: return launch_decode_d<128>(a, stage, stream);
        case 256: return launch_decode_d<256>(a, stage, stream);
        default: return 1;
    }
}

int decode_wg_tokens(int head_dim, int kv_heads_per_group)
{
    const int lps = head_dim == 64 ? 4 : (head_dim == 256 ? 16 : 8);
    const int spw = kWave / lps;
    return kTB * (spw / kv_heads_per_group) * kDecodeWaves;
}

void launch_splitkv_combine_rows(const float* partial_out, const float* partial_ml, const int64_t* piece_begin,
                                 const int64_t* piece_end, int64_t rows, int64_t head_dim, void* output,
                                 hipStream_t stream)
{
    hipLaunchKernelGGL(splitkv_combine_rows_kernel, dim3((unsigned)rows), dim3(64), 0, stream, partial_out, partial_ml,
                       piece_begin, piece_end, head_dim, (half_t*)output);
}

} // namespace pmxhip
