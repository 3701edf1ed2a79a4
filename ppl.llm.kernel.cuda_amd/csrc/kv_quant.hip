// KV-cache quantise/append for gfx950: fp16 K/V -> symmetric int8 in groups of 8
// channels with one fp16 scale per group, scattered into the cache.
//
// Arithmetic restated from the reference kernel
// (src/ppl/kernel/llm/cuda/pmx/multi_head_cache_attention/kernel.cu:128-154):
//   absmax over the group in half; scale = half(float(absmax) / 127.0f);
//   scale = scale > eps ? scale : eps with eps = half(1e-5f) (a half subnormal);
//   q = (int8) round-half-even( half(x / scale) ).
// The half quotient is the correctly rounded binary32 quotient rounded once more to
// binary16, which equals the correctly rounded half quotient (24 >= 2*11 + 2); the
// binary32 quotient comes from one division per group (the reciprocal of the scale) and
// a residual correction per element, see quantise_group.  The integer rounding is an
// addition in half (1536 + h, ulp one) -- HIP's __half2short_rn truncates, so it is not used.
//
// Decomposition (this file's own): a flat grid over (new token, group of 8
// channels); one lane owns one group of K and the same group of V: two 128-bit
// loads, two 64-bit int8 stores, two 16-bit scale stores.  The sequence of a
// token is found by bisection over seqstarts, so no workgroup is launched per
// (position, sequence) pair that does not exist.
#include <cmath>

#include "device_common.h"
#include "launch_params.h"

namespace pmxhip {

namespace {

constexpr int kQuantThreads = 256;

struct Quantised {
    u32x2 q;
    half_t scale;
};

// float(h.x) * b + c and float(h.y) * b + c with the half operand read in place (one instruction, one rounding)
__device__ __forceinline__ float fma_half_lo(half2_t h, float b, float c)
{
    float r;
    asm("v_fma_mix_f32 %0, %1, %2, %3 op_sel_hi:[1,0,0]" : "=v"(r) : "v"(h), "v"(b), "v"(c));
    return r;
}
__device__ __forceinline__ float fma_half_hi(half2_t h, float b, float c)
{
    float r;
    asm("v_fma_mix_f32 %0, %1, %2, %3 op_sel:[1,0,0] op_sel_hi:[1,0,0]" : "=v"(r) : "v"(h), "v"(b), "v"(c));
    return r;
}
// float(h.x) - a * b and float(h.y) - a * b (the negation is a source modifier)
__device__ __forceinline__ float half_lo_minus_product(half2_t h, float a, float b)
{
    float r;
    asm("v_fma_mix_f32 %0, -%1, %2, %3 op_sel_hi:[0,0,1]" : "=v"(r) : "v"(a), "v"(b), "v"(h));
    return r;
}
__device__ __forceinline__ float half_hi_minus_product(half2_t h, float a, float b)
{
    float r;
    asm("v_fma_mix_f32 %0, -%1, %2, %3 op_sel:[0,0,1] op_sel_hi:[0,0,1]" : "=v"(r) : "v"(a), "v"(b), "v"(h));
    return r;
}

__device__ __forceinline__ Quantised quantise_group(const u32x4 raw)
{
    half2_t x[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) x[i] = bitcast<half2_t>(raw[i]);
    // absmax in half, two channels at a time (sign bits cleared, packed maximum), then the two halves of the result
    half2_t m2 = bitcast<half2_t>(raw[0] & 0x7fff7fffu);
#pragma unroll
    for (int i = 1; i < 4; ++i) m2 = __builtin_elementwise_max(m2, bitcast<half2_t>(raw[i] & 0x7fff7fffu));
    const half_t amax = m2.x > m2.y ? m2.x : m2.y;
    const half_t eps = (half_t)1e-5f;
    // float(amax) / 127.0f, correctly rounded, without the division sequence: with r = fl(1 / 127), q0 = a * r,
    // e = fma(-q0, 127, a), q = fma(e, r, q0).  Equal to the correctly rounded quotient for every positive finite
    // half a (all 31 743 compared in exact arithmetic on the CPU).
    const float af = (float)amax;
    const float r127 = 1.0f / 127.0f;
    const float s0 = af * r127;
    half_t s = (half_t)__builtin_fmaf(__builtin_fmaf(-s0, 127.0f, af), r127, s0);
    s = s > eps ? s : eps;
    const float sf = (float)s;
    // One correctly rounded reciprocal per group, then a residual step per element:
    //   q0 = x * rcp, e = fma(-q0, sf, x), quotient = fma(e, rcp, q0).
    // Rounded to half this equals the correctly rounded quotient for every pair of a finite half x and a half
    // scale >= eps (all 2.0e9 pairs compared on the CPU; the one difference, -0 / s -> +0, yields the same int8 0).
    // The half channels enter the mixed-precision multiply-adds in place, two quotients are rounded to half by one
    // packed conversion, and the integer rounding is an addition: 1536 + h in half has an ulp of one, so the sum
    // is h rounded to the nearest integer with ties to even, and its low byte is that integer in two's
    // complement (|h| <= 127.4, the sum stays inside [1024, 2048)).
    const float rcp = 1.0f / sf;
    const half2_t magic = {(half_t)1536.0f, (half_t)1536.0f};
    uint32_t biased[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const float a0 = fma_half_lo(x[i], rcp, 0.0f), a1 = fma_half_hi(x[i], rcp, 0.0f);
        const float e0 = half_lo_minus_product(x[i], a0, sf), e1 = half_hi_minus_product(x[i], a1, sf);
        const float q0 = __builtin_fmaf(e0, rcp, a0), q1 = __builtin_fmaf(e1, rcp, a1);
        typedef float float2_t __attribute__((ext_vector_type(2)));
        const half2_t h = __builtin_convertvector(float2_t{q0, q1}, half2_t); // round to nearest even, both at once
        biased[i] = bitcast<uint32_t>(h + magic);
    }
    Quantised r;
    // bytes 0 and 2 of each word are the integers of its two channels
    r.q = u32x2{__builtin_amdgcn_perm(biased[1], biased[0], 0x06040200u), __builtin_amdgcn_perm(biased[3], biased[2], 0x06040200u)};
    r.scale = s;
    return r;
}

// largest b in [0, n) with starts[b] <= v   (starts non-decreasing, starts[0] <= v < starts[n]);
// being the largest, it is never an empty sequence
template <typename PTR>
__device__ __forceinline__ int sequence_of(PTR starts, int n, int64_t v)
{
    int lo = 0, hi = n - 1;
    while (lo < hi) {
        const int mid = (lo + hi + 1) >> 1;
        if (starts[mid] <= v) lo = mid;
        else hi = mid - 1;
    }
    return lo;
}

// The same index found by the wave's lanes together: the number of sequences that end at or before v (every lane
// of the wave must be here, with the same v).  Each lane compares one entry per 64, all requested at once: one
// memory latency where the bisection has log2(n) of them in a row.
constexpr int kCountedSequences = 1024;
__device__ __forceinline__ int sequence_by_count(const int64_t* starts, int n, int64_t v, int lane)
{
    int count = 0;
    for (int i0 = 0; i0 < n; i0 += kWave) {
        const int i = i0 + lane;
        const bool ends_before = i < n && starts[i + 1] <= v;
        count += __builtin_popcountll(__builtin_amdgcn_ballot_w64(ends_before));
    }
    return count < n ? count : n - 1;
}

} // namespace

// stride_tokens: tokens between a thread's units, (workgroups * threads) / groups_per_token; the host sizes the launch
// so that this division is exact whenever a thread takes more than one unit, which keeps a thread on one
// (head, channel group) for all its units: the two integer divisions below then happen once, not once per unit.
// WAVE_TOKEN: a token row has a multiple of 64 groups, so the 64 lanes of a wave always work on one token: what
// follows from the token alone (its sequence, position, cache row and the row bases) is then found once per wave
// on the scalar unit, with scalar loads of the index arrays, and a lane adds only its offset inside the row.
template <bool PAGED, bool WAVE_TOKEN>
__global__ __launch_bounds__(kQuantThreads) void kv_quantize_kernel(const QuantLaunch a, const uint32_t stride_tokens)
{
    const uint32_t groups_per_head = (uint32_t)a.head_dim >> 3;
    const uint32_t groups_per_token = (uint32_t)a.num_kv_heads * groups_per_head;
    const const_i64_ptr seqstarts = as_constant(a.seqstarts);
    const const_i64_ptr start_pos = as_constant(a.start_pos);
    const const_i64_ptr cachestarts = as_constant(a.cachestarts);
    const int64_t first = seqstarts[0];
    const int64_t n_tokens = seqstarts[a.batch] - first;
    const uint32_t u0 = blockIdx.x * kQuantThreads + threadIdx.x; // the host keeps workgroups * threads below 2^31
    uint32_t tok0 = u0 / groups_per_token;
    const uint32_t gi = u0 - tok0 * groups_per_token;
    if (WAVE_TOKEN) tok0 = __builtin_amdgcn_readfirstlane(tok0);
    const uint32_t h = gi / groups_per_head;
    const uint32_t d0 = (gi - h * groups_per_head) << 3;
    const uint32_t in_idx = h * (uint32_t)a.head_dim + d0;                   // halves inside a K/V row
    const int64_t out_idx = a.layer_idx * a.cache_stride_l + (int64_t)h * a.cache_stride_h + d0;
    for (int64_t tok = tok0; tok < n_tokens; tok += stride_tokens) {
        const int64_t in_tok = first + tok;
        // the rows to quantise do not depend on the sequence: requested first, they travel during the index lookups
        const u32x4 kraw = *(const u32x4*)((const half_t*)a.current_key + in_tok * a.current_key_stride_s + in_idx);
        const u32x4 vraw = *(const u32x4*)((const half_t*)a.current_value + in_tok * a.current_value_stride_s + in_idx);
        // decode steps have one new token per sequence: token i then belongs to sequence i, which two independent
        // loads confirm; otherwise the sequence is found by bisection (a chain of dependent loads)
        // (the sequence's start_pos is requested together with them, so that the decode step's chain of dependent
        // loads is index arrays -> page table -> stores)
        int b;
        int64_t pos;
        const int64_t ti = tok < a.batch ? tok : 0;
        const int64_t s0 = seqstarts[ti], s1 = seqstarts[ti + 1], sp = start_pos[ti];
        if (tok < a.batch && s0 == in_tok && s1 > in_tok) {
            b = (int)tok;
            pos = sp;
        } else {
            b = sequence_of(seqstarts, (int)a.batch, in_tok);
            pos = start_pos[b] + (in_tok - seqstarts[b]);
        }
        const int64_t tb = PAGED ? (int64_t)b * a.cachestarts_stride_b : (int64_t)b;
        const int64_t row = PAGED ? cachestarts[tb + (pos >> 7)] + (pos & (kPage - 1)) : cachestarts[tb] + pos;

        const Quantised kq = quantise_group(kraw);
        const Quantised vq = quantise_group(vraw);

        const int64_t k_out = row * a.cache_stride_s + out_idx;
        const int64_t v_out = k_out + a.cache_stride_kv;
        // Non-temporal: a wave writes whole lines (16 lanes x 8 bytes per row of a head, 64 scales), nothing here
        // reads them again, and lines left dirty in the memory-side cache are written back during the kernel that
        // runs next: the decode launch behind a prefill step's append (28 MB of rows) then took 17 us longer.
        __builtin_nontemporal_store(kq.q, (u32x2*)(a.cache + k_out));
        __builtin_nontemporal_store(vq.q, (u32x2*)(a.cache + v_out));
        __builtin_nontemporal_store(kq.scale, &((half_t*)a.scale)[k_out >> 3]);
        __builtin_nontemporal_store(vq.scale, &((half_t*)a.scale)[v_out >> 3]);
    }
}

// Rotary position embedding of Q and K (interleaved pairs, reference:
// src/ppl/kernel/llm/cuda/pmx/rotary_position_embedding.cu:35-91, 268-343), optionally fused with the
// quantise/append above: one workgroup per new token; the cos/sin of the token's position are computed
// once per pair (not once per head) and shared through LDS; a lane then rotates one group of 8 channels
// of a query head, or rotates and quantises the same group of K and quantises that of V.
//
// Angle (one definition for device and CPU): inv = 1.0f / float(pow(theta', i / (rotary_dim / 2)));
// angle = inv * float(pos) (linear scaling: inv * (float(pos) / factor)); cos and sin are those of the
// binary32 angle, correctly rounded to binary32 (evaluated in binary64).  The reference evaluates the
// same formula with the approximate __powf / __sincosf intrinsics.
template <bool PAGED>
__global__ __launch_bounds__(kQuantThreads) void rope_append_kernel(const RopeLaunch a)
{
    // a workgroup takes as many consecutive tokens as its threads can compute coefficients for in one go
    __shared__ float s_cos[kQuantThreads], s_sin[kQuantThreads];
    __shared__ int64_t s_row[kQuantThreads / 4];
    const int pairs = a.head_dim >> 1, rd2 = a.rotary_dim >> 1;
    const int tokens_per_wg = a.tokens_per_wg; // at most kQuantThreads / pairs; pairs <= 128
    const int64_t first = a.seqstarts[0];
    const int64_t n_tokens = a.seqstarts[a.batch] - first;
    const int64_t tok0 = (int64_t)blockIdx.x * tokens_per_wg;
    if (tok0 >= n_tokens) return;
    const bool append = a.cache != nullptr;

    // the rows of this workgroup's tokens, as units of 8 channels: the query heads' groups, then the key heads' (a
    // key unit also carries the same group of V when the step appends)
    const int gph = a.head_dim >> 3; // groups of 8 channels per head
    const int q_units = (int)a.num_heads * gph;
    const int k_units = (int)a.num_key_heads * gph;
    const int units = q_units + k_units;
    int n_here = tokens_per_wg;
    if (tok0 + n_here > n_tokens) n_here = (int)(n_tokens - tok0);
    const int work = n_here * units;

    struct Unit {
        int tl, h, d0;
        bool is_query;
        int64_t in_tok, idx;
    };
    auto unit_of = [&](int w) -> Unit {
        Unit r;
        r.tl = w / units;
        int u = w - r.tl * units;
        r.is_query = u < q_units;
        if (!r.is_query) u -= q_units;
        r.h = u / gph;
        r.d0 = (u - r.h * gph) << 3;
        r.in_tok = first + tok0 + r.tl;
        r.idx = (int64_t)r.h * a.head_dim + r.d0;
        return r;
    };
    auto load_row = [&](const Unit& r) -> u32x4 {
        return r.is_query ? *(const u32x4*)((const half_t*)a.query + r.in_tok * a.query_stride_s + r.idx)
                          : *(const u32x4*)((const half_t*)a.key + r.in_tok * a.key_stride_s + r.idx);
    };
    auto load_value = [&](const Unit& r) -> u32x4 {
        return *(const u32x4*)((const half_t*)a.value + r.in_tok * a.value_stride_s + r.idx);
    };

    // The rows depend on nothing that follows (index arrays -> sequence -> cos/sin and cache row), so a thread's
    // first units are requested before all that and travel meanwhile; a decode step, with a token per workgroup
    // and a few units per thread, has no others.
    constexpr int kEarly = 3;
    u32x4 early_row[kEarly], early_value[kEarly];
#pragma unroll
    for (int j = 0; j < kEarly; ++j) {
        const int w = threadIdx.x + j * kQuantThreads;
        early_row[j] = u32x4{0, 0, 0, 0};
        early_value[j] = u32x4{0, 0, 0, 0};
        if (w < work) {
            const Unit r = unit_of(w);
            early_row[j] = load_row(r);
            if (append && !r.is_query) early_value[j] = load_value(r);
        }
    }

    {
        const int tl = threadIdx.x / pairs, i = threadIdx.x - tl * pairs;
        const int64_t tok = tok0 + tl;
        const bool active = tl < tokens_per_wg && tok < n_tokens;
        const int64_t in_tok = first + tok;
        // The token's sequence.  One new token per sequence (a decode step): token i belongs to sequence i, which two
        // independent loads confirm.  Otherwise the lanes of the wave count, for each token the wave covers, the
        // sequences that end before it (one latency); beyond kCountedSequences sequences every thread bisects (a
        // chain of dependent loads).
        int b = -1;
        int64_t pos = 0;
        const bool count_search = a.batch <= kCountedSequences;
        if (active && (n_tokens == a.batch || !count_search)) {
            const int64_t ti = tok < a.batch ? tok : 0;
            const int64_t s0 = a.seqstarts[ti], s1 = a.seqstarts[ti + 1], sp = a.start_pos[ti];
            if (tok < a.batch && s0 == in_tok && s1 > in_tok) {
                b = (int)tok;
                pos = sp;
            }
        }
        if (count_search) { // every lane of the wave is here
            const int wave0 = threadIdx.x & ~(kWave - 1);
            const int tl_hi = (wave0 + kWave - 1) / pairs;
            for (int t = wave0 / pairs; t <= tl_hi; ++t) {
                const int64_t tk = tok0 + t;
                if (t >= tokens_per_wg || tk >= n_tokens) break;
                if (__builtin_amdgcn_ballot_w64(tl == t && b < 0) == 0) continue;
                const int bt = sequence_by_count(a.seqstarts, (int)a.batch, first + tk, threadIdx.x & (kWave - 1));
                if (tl == t && b < 0) {
                    b = bt;
                    pos = a.start_pos[bt] + (first + tk - a.seqstarts[bt]);
                }
            }
        } else if (active && b < 0) {
            b = sequence_of(a.seqstarts, (int)a.batch, in_tok);
            pos = a.start_pos[b] + (in_tok - a.seqstarts[b]);
        }
        if (active) {
            float c = 1.f, s = 0.f;
            if (i < rd2) {
                float th = a.theta;
                if (a.scaling_type == 2) { // dynamic: rotary_position_embedding.cu:68-91
                    const int64_t pos_end = a.start_pos[b] + (a.seqstarts[b + 1] - a.seqstarts[b]);
                    if (pos_end > a.max_position_embeddings) {
                        const float base = ((a.scaling_factor * (float)pos_end) / (float)a.max_position_embeddings) - (a.scaling_factor - 1.f);
                        const float expn = (float)rd2 / (float)(rd2 - 1);
                        th = a.theta * (float)pow((double)base, (double)expn);
                    }
                }
                // theta^(i / rd2) is the same for every token unless the dynamic scaling applies: then it comes in the
                // launch arguments and the binary64 pow leaves the kernel
                const float inv = a.has_inv_freq ? a.inv_freq[i] : 1.0f / (float)pow((double)th, (double)((float)i / (float)rd2));
                const float p = a.scaling_type == 1 ? (float)pos / a.scaling_factor : (float)pos;
                const float angle = inv * p;
                double sd, cd;
                sincos((double)angle, &sd, &cd); // one argument reduction for both
                c = (float)cd;
                s = (float)sd;
            }
            s_cos[threadIdx.x] = c;
            s_sin[threadIdx.x] = s;
            if (i == 0 && append)
                s_row[tl] = token_row<PAGED>(a.cachestarts, PAGED ? (int64_t)b * a.cachestarts_stride_b : (int64_t)b, pos);
        }
    }
    __syncthreads();

    auto rotate = [&](const u32x4 raw, int d0, int tl) -> u32x4 {
        u32x4 out;
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            const int i = (d0 >> 1) + w;
            const half2_t h = bitcast<half2_t>(raw[w]);
            if (i < rd2) {
                const float x = (float)h.x, y = (float)h.y, c = s_cos[tl * pairs + i], s = s_sin[tl * pairs + i];
                const half2_t r = {(half_t)(x * c - y * s), (half_t)(y * c + x * s)};
                out[w] = bitcast<uint32_t>(r);
            } else {
                out[w] = raw[w];
            }
        }
        return out;
    };

    auto finish = [&](const Unit& r, u32x4 raw, const u32x4 vraw) {
        if (r.is_query) {
            *(u32x4*)((half_t*)a.rotated_query + r.in_tok * a.rotated_query_stride_s + r.idx) = rotate(raw, r.d0, r.tl);
            return;
        }
        if (!a.bypass_key) raw = rotate(raw, r.d0, r.tl);
        if (a.rotated_key) *(u32x4*)((half_t*)a.rotated_key + r.in_tok * a.rotated_key_stride_s + r.idx) = raw;
        if (append) {
            const Quantised kq = quantise_group(raw);
            const Quantised vq = quantise_group(vraw);
            const int64_t k_out = s_row[r.tl] * a.cache_stride_s + a.layer_idx * a.cache_stride_l + (int64_t)r.h * a.cache_stride_h + r.d0;
            const int64_t v_out = k_out + a.cache_stride_kv;
            __builtin_nontemporal_store(kq.q, (u32x2*)(a.cache + k_out));
            __builtin_nontemporal_store(vq.q, (u32x2*)(a.cache + v_out));
            __builtin_nontemporal_store(kq.scale, &((half_t*)a.scale)[k_out >> 3]);
            __builtin_nontemporal_store(vq.scale, &((half_t*)a.scale)[v_out >> 3]);
        }
    };

#pragma unroll
    for (int j = 0; j < kEarly; ++j) {
        const int w = threadIdx.x + j * kQuantThreads;
        if (w < work) finish(unit_of(w), early_row[j], early_value[j]);
    }
    for (int w = threadIdx.x + kEarly * kQuantThreads; w < work; w += kQuantThreads) {
        const Unit r = unit_of(w);
        const u32x4 raw = load_row(r);
        u32x4 vraw = {0, 0, 0, 0};
        if (append && !r.is_query) vraw = load_value(r);
        finish(r, raw, vraw);
    }
}

int launch_rope(const RopeLaunch& a_in, int compute_units, hipStream_t stream)
{
    if (a_in.max_tokens <= 0) return kLaunchOk;
    if (a_in.head_dim > 256 || a_in.head_dim < 8) return kLaunchNoKernel;
    RopeLaunch a = a_in;
    const int pairs = a.head_dim / 2, rd2 = a.rotary_dim / 2;
    a.has_inv_freq = 0;
    if (a.scaling_type != 2 && rd2 <= 128) {
        for (int i = 0; i < rd2; ++i) a.inv_freq[i] = 1.0f / (float)pow((double)a.theta, (double)((float)i / (float)rd2));
        a.has_inv_freq = 1;
    }
    // A workgroup computes the coefficients of its tokens once and shares them through LDS: as many tokens as its
    // threads have pairs for, but no more than leaves two workgroups per CU (a decode step has a token per sequence,
    // and a workgroup works through its tokens' rows one after the other)
    int tokens_per_wg = kQuantThreads / pairs;
    const int64_t spread = a.max_tokens / (2 * (int64_t)(compute_units > 0 ? compute_units : 256));
    if (tokens_per_wg > spread) tokens_per_wg = spread > 1 ? (int)spread : 1;
    a.tokens_per_wg = tokens_per_wg;
    const unsigned blocks = (unsigned)((a.max_tokens + tokens_per_wg - 1) / tokens_per_wg);
    if (a.cache_mode == 1) hipLaunchKernelGGL(rope_append_kernel<true>, dim3(blocks), dim3(kQuantThreads), 0, stream, a);
    else hipLaunchKernelGGL(rope_append_kernel<false>, dim3(blocks), dim3(kQuantThreads), 0, stream, a);
    return kLaunchOk;
}

int launch_kv_quantize(const QuantLaunch& a, int compute_units, hipStream_t stream)
{
    const int64_t groups_per_token = (int64_t)a.num_kv_heads * (a.head_dim >> 3);
    const int64_t max_units = a.max_tokens * groups_per_token;
    if (max_units <= 0) return kLaunchOk;
    int64_t blocks = (max_units + kQuantThreads - 1) / kQuantThreads;
    // grid-stride beyond this: eight workgroups per CU hold every wave slot at once, and a lane then takes two or
    // three units in turn (11 104 new tokens of 8 heads x 128 channels on 256 CUs: 23.4 us against 28 us with four
    // times as many workgroups and one unit per lane, 36 us with 32 times as many, most of them without a unit;
    // 25 us with half as many)
    const int64_t cap = (int64_t)(compute_units > 0 ? compute_units : 256) * 8;
    if (blocks > cap) {
        // a whole number of token rows per sweep of the grid, so that a thread keeps its (head, channel group):
        // the workgroup count is a multiple of groups_per_token / gcd(groups_per_token, threads per workgroup)
        int64_t g = groups_per_token, t = kQuantThreads;
        while (t != 0) {
            const int64_t r = g % t;
            g = t;
            t = r;
        }
        const int64_t unit = groups_per_token / g;
        blocks = cap / unit * unit;
        if (blocks == 0) blocks = unit;
    }
    if (blocks * kQuantThreads >= (int64_t)1 << 31) return kLaunchNoKernel;
    // exact when blocks was rounded above; otherwise no thread takes a second unit and the value only has to carry
    // a thread beyond the last token
    const uint32_t stride_tokens = (uint32_t)((blocks * kQuantThreads + groups_per_token - 1) / groups_per_token);
    const bool wave_token = groups_per_token % kWave == 0;
    const dim3 grid((unsigned)blocks), block(kQuantThreads);
    if (a.cache_mode == 1) {
        if (wave_token) hipLaunchKernelGGL((kv_quantize_kernel<true, true>), grid, block, 0, stream, a, stride_tokens);
        else hipLaunchKernelGGL((kv_quantize_kernel<true, false>), grid, block, 0, stream, a, stride_tokens);
    } else {
        if (wave_token) hipLaunchKernelGGL((kv_quantize_kernel<false, true>), grid, block, 0, stream, a, stride_tokens);
        else hipLaunchKernelGGL((kv_quantize_kernel<false, false>), grid, block, 0, stream, a, stride_tokens);
    }
    return kLaunchOk;
}

} // namespace pmxhip
