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
// a residual correction per element, see quantise_group.  The integer rounding is
// v_rndne -- HIP's __half2short_rn truncates, so it is not used.
//
// Decomposition (this file's own): a flat grid over (new token, group of 8
// channels); one lane owns one group of K and the same group of V: two 128-bit
// loads, two 64-bit int8 stores, two 16-bit scale stores.  The sequence of a
// token is found by bisection over seqstarts, so no workgroup is launched per
// (position, sequence) pair that does not exist.
#include "device_common.h"
#include "launch_params.h"

namespace pmxhip {

namespace {

constexpr int kQuantThreads = 256;

struct Quantised {
    u32x2 q;
    half_t scale;
};

__device__ __forceinline__ Quantised quantise_group(const u32x4 raw)
{
    half_t x[8];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const half2_t h = bitcast<half2_t>(raw[i]);
        x[2 * i] = h.x;
        x[2 * i + 1] = h.y;
    }
    half_t amax = (half_t)0.0f;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const half_t ax = __builtin_fabsf16(x[i]);
        amax = amax > ax ? amax : ax;
    }
    const half_t eps = (half_t)1e-5f;
    half_t s = (half_t)((float)amax / 127.0f);
    s = s > eps ? s : eps;
    const float sf = (float)s;
    // One correctly rounded reciprocal per group, then a residual step per element:
    //   q0 = x * rcp, e = fma(-q0, sf, x), quotient = fma(e, rcp, q0).
    // Rounded to half this equals the correctly rounded quotient for every pair of a finite half x and a half
    // scale >= eps (all 2.0e9 pairs compared on the CPU; the one difference, -0 / s -> +0, yields the same int8 0).
    const float rcp = 1.0f / sf;
    uint32_t packed[2] = {0u, 0u};
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const float xf = (float)x[i];
        const float q0 = xf * rcp;
        const half_t quo = (half_t)__builtin_fmaf(__builtin_fmaf(-q0, sf, xf), rcp, q0);
        const int qi = (int)__builtin_rintf((float)quo);
        packed[i >> 2] |= ((uint32_t)qi & 0xffu) << (8 * (i & 3));
    }
    Quantised r;
    r.q = u32x2{packed[0], packed[1]};
    r.scale = s;
    return r;
}

// largest b in [0, n) with starts[b] <= v   (starts non-decreasing, starts[0] <= v < starts[n]);
// being the largest, it is never an empty sequence
__device__ __forceinline__ int sequence_of(const int64_t* __restrict__ starts, int n, int64_t v)
{
    int lo = 0, hi = n - 1;
    while (lo < hi) {
        const int mid = (lo + hi + 1) >> 1;
        if (starts[mid] <= v) lo = mid;
        else hi = mid - 1;
    }
    return lo;
}

} // namespace

template <bool PAGED>
__global__ __launch_bounds__(kQuantThreads) void kv_quantize_kernel(const QuantLaunch a)
{
    const int groups_per_head = a.head_dim >> 3;
    const int groups_per_token = a.num_kv_heads * groups_per_head;
    const int64_t first = a.seqstarts[0];
    const int64_t n_tokens = a.seqstarts[a.batch] - first;
    const int64_t n_units = n_tokens * groups_per_token;
    const int64_t stride = (int64_t)gridDim.x * kQuantThreads;
    for (int64_t u = (int64_t)blockIdx.x * kQuantThreads + threadIdx.x; u < n_units; u += stride) {
        const int64_t tok = u / groups_per_token;
        const int gi = (int)(u - tok * groups_per_token);
        const int h = gi / groups_per_head;
        const int d0 = (gi - h * groups_per_head) << 3;
        const int64_t in_tok = first + tok;
        // the rows to quantise do not depend on the sequence: requested first, they travel during the index lookups
        const int64_t in_idx = (int64_t)h * a.head_dim + d0;
        const u32x4 kraw = *(const u32x4*)((const half_t*)a.current_key + in_tok * a.current_key_stride_s + in_idx);
        const u32x4 vraw = *(const u32x4*)((const half_t*)a.current_value + in_tok * a.current_value_stride_s + in_idx);
        // decode steps have one new token per sequence: token i then belongs to sequence i, which two independent
        // loads confirm; otherwise the sequence is found by bisection (a chain of dependent loads)
        // (the sequence's start_pos is requested together with them, so that the decode step's chain of dependent
        // loads is index arrays -> page table -> stores)
        int b;
        int64_t pos;
        const int64_t ti = tok < a.batch ? tok : 0;
        const int64_t s0 = a.seqstarts[ti], s1 = a.seqstarts[ti + 1], sp = a.start_pos[ti];
        if (tok < a.batch && s0 == in_tok && s1 > in_tok) {
            b = (int)tok;
            pos = sp;
        } else {
            b = sequence_of(a.seqstarts, (int)a.batch, in_tok);
            pos = a.start_pos[b] + (in_tok - a.seqstarts[b]);
        }
        const int64_t row = token_row<PAGED>(a.cachestarts, PAGED ? (int64_t)b * a.cachestarts_stride_b : (int64_t)b, pos);

        const Quantised kq = quantise_group(kraw);
        const Quantised vq = quantise_group(vraw);

        const int64_t k_out = row * a.cache_stride_s + a.layer_idx * a.cache_stride_l + (int64_t)h * a.cache_stride_h + d0;
        const int64_t v_out = k_out + a.cache_stride_kv;
        *(u32x2*)(a.cache + k_out) = kq.q;
        *(u32x2*)(a.cache + v_out) = vq.q;
        ((half_t*)a.scale)[k_out >> 3] = kq.scale;
        ((half_t*)a.scale)[v_out >> 3] = vq.scale;
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
    const int tokens_per_wg = kQuantThreads / pairs; // pairs <= 128
    const int64_t first = a.seqstarts[0];
    const int64_t n_tokens = a.seqstarts[a.batch] - first;
    const int64_t tok0 = (int64_t)blockIdx.x * tokens_per_wg;
    if (tok0 >= n_tokens) return;
    const bool append = a.cache != nullptr;

    {
        const int tl = threadIdx.x / pairs, i = threadIdx.x - tl * pairs;
        const int64_t tok = tok0 + tl;
        if (tl < tokens_per_wg && tok < n_tokens) {
            const int64_t in_tok = first + tok;
            const int b = sequence_of(a.seqstarts, (int)a.batch, in_tok);
            const int64_t pos = a.start_pos[b] + (in_tok - a.seqstarts[b]);
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
                const float inv = 1.0f / (float)pow((double)th, (double)((float)i / (float)rd2));
                const float p = a.scaling_type == 1 ? (float)pos / a.scaling_factor : (float)pos;
                const float angle = inv * p;
                c = (float)cos((double)angle);
                s = (float)sin((double)angle);
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

    const int gph = a.head_dim >> 3; // groups of 8 channels per head
    const int q_units = (int)a.num_heads * gph;
    const int k_units = (int)a.num_key_heads * gph;
    const int units = q_units + k_units;
    int n_here = tokens_per_wg;
    if (tok0 + n_here > n_tokens) n_here = (int)(n_tokens - tok0);
    for (int w = threadIdx.x; w < n_here * units; w += kQuantThreads) {
        const int tl = w / units, u = w - tl * units;
        const int64_t in_tok = first + tok0 + tl;
        if (u < q_units) {
            const int h = u / gph, d0 = (u - h * gph) << 3;
            const int64_t idx = (int64_t)h * a.head_dim + d0;
            const u32x4 raw = *(const u32x4*)((const half_t*)a.query + in_tok * a.query_stride_s + idx);
            *(u32x4*)((half_t*)a.rotated_query + in_tok * a.rotated_query_stride_s + idx) = rotate(raw, d0, tl);
        } else {
            const int uk = u - q_units;
            const int h = uk / gph, d0 = (uk - h * gph) << 3;
            const int64_t idx = (int64_t)h * a.head_dim + d0;
            u32x4 kraw = *(const u32x4*)((const half_t*)a.key + in_tok * a.key_stride_s + idx);
            if (!a.bypass_key) kraw = rotate(kraw, d0, tl);
            if (a.rotated_key) *(u32x4*)((half_t*)a.rotated_key + in_tok * a.rotated_key_stride_s + idx) = kraw;
            if (append) {
                const u32x4 vraw = *(const u32x4*)((const half_t*)a.value + in_tok * a.value_stride_s + idx);
                const Quantised kq = quantise_group(kraw);
                const Quantised vq = quantise_group(vraw);
                const int64_t k_out = s_row[tl] * a.cache_stride_s + a.layer_idx * a.cache_stride_l + (int64_t)h * a.cache_stride_h + d0;
                const int64_t v_out = k_out + a.cache_stride_kv;
                *(u32x2*)(a.cache + k_out) = kq.q;
                *(u32x2*)(a.cache + v_out) = vq.q;
                ((half_t*)a.scale)[k_out >> 3] = kq.scale;
                ((half_t*)a.scale)[v_out >> 3] = vq.scale;
            }
        }
    }
}

int launch_rope(const RopeLaunch& a, hipStream_t stream)
{
    if (a.max_tokens <= 0) return 0;
    if (a.head_dim > 256 || a.head_dim < 8) return 1;
    const int tokens_per_wg = kQuantThreads / (a.head_dim / 2);
    const unsigned blocks = (unsigned)((a.max_tokens + tokens_per_wg - 1) / tokens_per_wg);
    if (a.cache_mode == 1) hipLaunchKernelGGL(rope_append_kernel<true>, dim3(blocks), dim3(kQuantThreads), 0, stream, a);
    else hipLaunchKernelGGL(rope_append_kernel<false>, dim3(blocks), dim3(kQuantThreads), 0, stream, a);
    return 0;
}

int launch_kv_quantize(const QuantLaunch& a, int compute_units, hipStream_t stream)
{
    const int64_t groups_per_token = (int64_t)a.num_kv_heads * (a.head_dim >> 3);
    const int64_t max_units = a.max_tokens * groups_per_token;
    if (max_units <= 0) return 0;
    int64_t blocks = (max_units + kQuantThreads - 1) / kQuantThreads;
    // grid-stride beyond this: eight workgroups per CU hold every wave slot at once, and a lane then takes two or
    // three units in turn (11 104 new tokens of 8 heads x 128 channels on 256 CUs: 23.4 us against 28 us with four
    // times as many workgroups and one unit per lane, 36 us with 32 times as many, most of them without a unit;
    // 25 us with half as many)
    const int64_t cap = (int64_t)(compute_units > 0 ? compute_units : 256) * 8;
    if (blocks > cap) blocks = cap;
    if (a.cache_mode == 1)
        hipLaunchKernelGGL(kv_quantize_kernel<true>, dim3((unsigned)blocks), dim3(kQuantThreads), 0, stream, a);
    else
        hipLaunchKernelGGL(kv_quantize_kernel<false>, dim3((unsigned)blocks), dim3(kQuantThreads), 0, stream, a);
    return 0;
}

} // namespace pmxhip
