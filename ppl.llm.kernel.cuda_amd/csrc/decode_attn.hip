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

constexpr int kDecodeThreads = 256;
constexpr int kDecodeWaves = kDecodeThreads / kWave;
constexpr int kTB = 4; // tokens a slot handles per block (= lanes of a quad)
static_assert(kTB == 4, "the quad reduce-scatter and the explicit wait counts assume four tokens per block");

// ---- hand-scheduled cache loads of the pipelined loop ---------------------------------------
// The loads of the steady-state loop are issued through inline assembly and awaited with explicit
// wait counts.  Written as plain C++ loads, the compiler's automatic wait-count placement reuses
// staging registers for temporaries and then waits for loads issued only moments earlier, which
// serialises the memory latency into every iteration.  Vector memory operations complete in issue
// order, so "at most N still outstanding" identifies exactly which loads have landed.
__device__ __forceinline__ void load_b128(u32x4& dst, uint32_t lane_off, const char* wave_base)
{
    asm volatile("global_load_dwordx4 %0, %1, %2" : "=&v"(dst) : "v"(lane_off), "s"(wave_base) : "memory");
}
__device__ __forceinline__ void load_b32(uint32_t& dst, uint32_t lane_off, const char* wave_base)
{
    asm volatile("global_load_dword %0, %1, %2" : "=&v"(dst) : "v"(lane_off), "s"(wave_base) : "memory");
}
// waits until at most N vector memory operations are outstanding; the values pass through the
// statement so that no use of them can be scheduled before the wait
template <int N>
__device__ __forceinline__ void wait_loads(u32x4& a, uint32_t& b)
{
    asm volatile("s_waitcnt vmcnt(%2)" : "+v"(a), "+v"(b) : "n"(N));
}
// Waits for every outstanding load.  A register that is the target of an in-flight load must stay
// allocated until a wait covers it, even when its value is never used (the redundant request of
// the last block): passing it through this statement keeps it reserved, so that nothing else can
// be placed in it and then be overwritten when the load lands.
__device__ __forceinline__ void drain_loads(u32x4 (&q)[4], uint32_t (&sc)[4])
{
    asm volatile("s_waitcnt vmcnt(0)"
                 : "+v"(q[0]), "+v"(q[1]), "+v"(q[2]), "+v"(q[3]), "+v"(sc[0]), "+v"(sc[1]), "+v"(sc[2]), "+v"(sc[3]));
}

// value held by quad lane (lane ^ j), j in 0..3; j is a compile-time constant after unrolling
__device__ __forceinline__ float quad_xor(float v, int j)
{
    switch (j) {
        case 0: return v;
        case 1: return dpp_f32<kDppXor1>(v);
        case 2: return dpp_f32<kDppXor2>(v);
        default: return dpp_f32<0x1B>(v); // quad_perm:[3,2,1,0]
    }
}

// Tokens per range: equal shares rounded up to a whole number of workgroup
// iterations, never below kMinTokensPerRange.  Shared by both kernels.
__device__ __forceinline__ int64_t tokens_per_range(int64_t total, int ranges, int wg_tokens, int min_tokens)
{
    int64_t per = (total + ranges - 1) / ranges;
    if (per < min_tokens) per = min_tokens;
    return (per + wg_tokens - 1) / wg_tokens * wg_tokens;
}

// first b in [0, n) with starts[b + 1] - starts[0] > g   (starts is non-decreasing)
__device__ __forceinline__ int find_sequence(const_i64_ptr starts, int n, int64_t g)
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

// One block of kTB tokens for one slot: raw cache bytes as loaded, K and V staged separately.
struct KBlock {
    u32x4 q8[kTB];    // 16 int8 key channels per token
    uint32_t sc[kTB]; // their two fp16 group scales
    int pos;          // sequence position of the wave block's first token
    int64_t boff;     // element offset of that token's row in the cache
};
struct VBlock {
    u32x4 q8[kTB];
    uint32_t sc[kTB];
};

// D: head dim (64, 96, 128, 256).  GT: query heads per kv head held in registers.
template <int D, int GT, bool PAGED, bool MASK>
__global__ __launch_bounds__(kDecodeThreads, (GT <= 4 ? 2 : 1)) void decode_attention_kernel(const DecodeLaunch a)
{
    constexpr int LPS = (D == 64) ? 4 : (D == 256 ? 16 : 8); // lanes per slot
    constexpr int LPS_ACTIVE = D / 16;                        // 6 of 8 for D = 96
    constexpr int SPW = kWave / LPS;                          // slots per wave
    constexpr int NSLOT = SPW * kDecodeWaves;
    constexpr bool kHandScheduled = GT <= 4; // inline-assembly loads with explicit wait counts in the steady-state loop

    __shared__ float sm_acc[NSLOT * D];
    __shared__ float sm_m[NSLOT];
    __shared__ float sm_l[NSLOT];

    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int ls = lane % LPS;            // lane in slot -> channels [16*ls, 16*ls+16)
    const int slot = lane / LPS;          // slot in wave
    // Token order inside a block is permuted per lane: register slot j of a lane holds token j ^ tp.
    // With tp = (lane in quad) ^ (3 on odd quads) the cross-lane sum of the four partial logits needs
    // no selects: slot k of a lane and slot k ^ 2 of its xor-2 partner are the same token, and so on
    // down to one complete logit per lane (token tp); the mirror partners used across quads own the
    // same token.  The probability of slot j's token is then found in quad lane (lane ^ j).
    const int tp = (lane & 3) ^ ((lane & 4) ? 3 : 0);
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

    const const_i64_ptr kvstarts = as_constant(a.kvstarts);
    const const_i64_ptr cachestarts = as_constant(a.cachestarts);
    const int64_t kv_base = kvstarts[0];
    const int64_t total = kvstarts[a.decoding_batches] - kv_base;
    const int64_t per = tokens_per_range(total, a.ranges, wg_tokens, a.min_tokens_per_range);
    const int64_t r0 = (int64_t)blockIdx.x * per;
    if (r0 >= total) return;
    const int64_t r1 = (r0 + per < total) ? r0 + per : total;
#ifdef PMX_WG_TRACE
    const unsigned long long trace_t0 = wall_clock64();
    const unsigned long long trace_c0 = clock64();
#endif

    // Addressing: a wave-uniform 64-bit base per block (scalar registers) plus a 32-bit per-lane
    // offset that never changes: (token in block) * stride_s + (head in group) * stride_h + channel.
    const int64_t group_off = a.layer_idx * a.cache_stride_l + (int64_t)(blockIdx.y * kvhb) * a.cache_stride_h;
    uint32_t voff[kTB];
#pragma unroll
    for (int j = 0; j < kTB; ++j)
        voff[j] = (uint32_t)((int64_t)((j ^ tp) * tpl + tsub) * a.cache_stride_s + (int64_t)head_local * a.cache_stride_h + ch0);
    uint32_t voff_sc[kTB]; // the same offsets in the scale tensor: one fp16 scale per 8 channels
#pragma unroll
    for (int j = 0; j < kTB; ++j) voff_sc[j] = voff[j] >> 2;
    const char* const cache_k = (const char*)a.cache + group_off;
    const char* const cache_v = cache_k + a.cache_stride_kv;
    const char* const scale_k = (const char*)a.scale + (group_off >> 3) * 2;
    const char* const scale_v = scale_k + (a.cache_stride_kv >> 3) * 2;
    const float logit_scale = a.attn_scale * kLog2e;

    int b = find_sequence(kvstarts, (int)a.decoding_batches, r0);
    for (; b < a.decoding_batches; ++b) {
        const int64_t s_beg = kvstarts[b] - kv_base;
        if (s_beg >= r1) break;
        const int64_t s_end = kvstarts[b + 1] - kv_base;
        const int64_t len = s_end - s_beg;
        // piece [pa, pe) in sequence coordinates
        const int64_t pa = (r0 > s_beg ? r0 : s_beg) - s_beg;
        const int64_t pe = (r1 < s_end ? r1 : s_end) - s_beg;
        if (pe <= pa) continue;

        // ---- query heads of this kv head into registers (packed halves) ----
        // qb[g][i] = -1152 * (sum of the 8 query channels of group i): the int8 -> half conversion
        // leaves keys biased by +1152 (see device_common.h); starting the dot product at qb removes
        // the bias exactly where it is cheapest.
        half2_t q[GT][8];
        float qb[GT][2];
#pragma unroll
        for (int g = 0; g < GT; ++g) {
            const int gi = g_first + g;
            const bool on = lane_on && gi < G;
            const int h = kvh * G + (gi < G ? gi : 0);
            const u32x4* qp = (const u32x4*)((const half_t*)a.query + (int64_t)b * a.query_stride_s + (int64_t)h * D + ch0);
            u32x4 lo = qp[0], hi = qp[1];
            if (!on) { lo = u32x4{0, 0, 0, 0}; hi = lo; }
            float s0 = 0.f, s1 = 0.f;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                q[g][i] = bitcast<half2_t>(lo[i]);
                q[g][4 + i] = bitcast<half2_t>(hi[i]);
                s0 += (float)q[g][i].x + (float)q[g][i].y;
                s1 += (float)q[g][4 + i].x + (float)q[g][4 + i].y;
            }
            qb[g][0] = -1152.f * s0;
            qb[g][1] = -1152.f * s1;
        }

        float m_run[GT], l_run[GT], acc[GT][16];
#pragma unroll
        for (int g = 0; g < GT; ++g) {
            m_run[g] = kNegBig;
            l_run[g] = 0.f; // partial: this lane's own tokens only
#pragma unroll
            for (int c = 0; c < 16; ++c) acc[g][c] = 0.f;
        }

        const int64_t table_base = PAGED ? (int64_t)b * a.cachestarts_stride_b : (int64_t)b;
        const int64_t seq_row0 = PAGED ? 0 : cachestarts[b];
        const half_t* mask_row = nullptr;
        if (MASK) mask_row = (const half_t*)a.attn_mask + (int64_t)b * a.mask_stride_s + kvstarts[b];
        // sequence-relative positions fit 32 bits
        const int pa32 = (int)pa, pe32 = (int)pe;
        const int last_page = (pe32 - 1) >> 7;

        // Page table entries are read one page ahead with scalar loads, so that no block waits
        // for its row base: `page_row` belongs to page `page_idx`, `next_row` to the page after it.
        int page_idx = -2;
        int64_t page_row = 0, next_row = 0;
        auto row_base_of = [&](int pos) -> int64_t {
            if (!PAGED) return seq_row0 + pos;
            const int pg = pos >> 7;
            if (pg != page_idx) {
                page_row = (pg == page_idx + 1) ? next_row : cachestarts[table_base + pg];
                page_idx = pg;
                const int nx = pg + 1 <= last_page ? pg + 1 : last_page;
                next_row = cachestarts[table_base + nx];
            }
            return page_row + (pos & (kPage - 1));
        };

        // ---- loads of one wave block (positions pos .. pos + wave_tokens): K with its scales, V with its scales.
        // FULL blocks lie inside the piece; in a partial block the tokens outside the piece are redirected
        // to a token inside it (the load is harmless, the logit is masked later) ----
        auto lane_off = [&](int pos, int j) -> uint32_t {
            const int t = pos + (j ^ tp) * tpl + tsub;
            const int tc = t < pa32 ? pa32 : (t >= pe32 ? pe32 - 1 : t);
            return (uint32_t)((int64_t)(tc - pos) * a.cache_stride_s + (int64_t)head_local * a.cache_stride_h + ch0);
        };
        // steady-state versions: full blocks only, inline-assembly loads in a fixed order
        // (token 0: 16 bytes then scales, token 1: ..., 8 operations per half-block)
        auto issue_k_fast = [&](KBlock& kb, int pos) {
            kb.pos = pos;
            const int64_t boff = row_base_of(pos) * a.cache_stride_s;
            kb.boff = boff;
            const char* bk = cache_k + boff;
            const char* sk = scale_k + (boff >> 3) * 2;
#pragma unroll
            for (int j = 0; j < kTB; ++j) {
                load_b128(kb.q8[j], voff[j], bk);
                load_b32(kb.sc[j], voff_sc[j], sk);
            }
        };
        auto issue_v_fast = [&](VBlock& vb, int64_t boff) {
            const char* bv = cache_v + boff;
            const char* sv = scale_v + (boff >> 3) * 2;
#pragma unroll
            for (int j = 0; j < kTB; ++j) {
                load_b128(vb.q8[j], voff[j], bv);
                load_b32(vb.sc[j], voff_sc[j], sv);
            }
        };
        auto issue_k = [&](KBlock& kb, int pos, bool full) {
            kb.pos = pos;
            const int64_t boff = row_base_of(pos) * a.cache_stride_s;
            kb.boff = boff;
            const char* bk = cache_k + boff;
            const char* sk = scale_k + (boff >> 3) * 2;
#pragma unroll
            for (int j = 0; j < kTB; ++j) {
                const uint32_t off = full ? voff[j] : lane_off(pos, j);
                kb.q8[j] = *(const u32x4*)(bk + off);
                kb.sc[j] = *(const uint32_t*)(sk + (off >> 2));
            }
        };
        auto issue_v = [&](VBlock& vb, int pos, int64_t boff, bool full) {
            const char* bv = cache_v + boff;
            const char* sv = scale_v + (boff >> 3) * 2;
#pragma unroll
            for (int j = 0; j < kTB; ++j) {
                const uint32_t off = full ? voff[j] : lane_off(pos, j);
                vb.q8[j] = *(const u32x4*)(bv + off);
                vb.sc[j] = *(const uint32_t*)(sv + (off >> 2));
            }
        };

        // ---- QK^T and softmax of one block: leaves this lane's probability (token ql) in p[g] ----
        float p[GT];
        auto logits_softmax = [&](KBlock& kb, bool full, bool fast) {
            // logits, still partial over the slot's lanes: part[g][j], log2 units
            float part[GT][kTB];
#pragma unroll
            for (int j = 0; j < kTB; ++j) {
                if (fast) {
                    // outstanding and younger than token j of this half-block: the rest of this half-block,
                    // and the two half-blocks requested after it
                    if (j == 0) wait_loads<22>(kb.q8[0], kb.sc[0]);
                    if (j == 1) wait_loads<20>(kb.q8[1], kb.sc[1]);
                    if (j == 2) wait_loads<18>(kb.q8[2], kb.sc[2]);
                    if (j == 3) wait_loads<16>(kb.q8[3], kb.sc[3]);
                }
                half2_t kh[8];
#pragma unroll
                for (int w = 0; w < 4; ++w) {
                    const uint32_t f = kb.q8[j][w] ^ kFlipSigns;
                    kh[2 * w] = bitcast<half2_t>(__builtin_amdgcn_perm(kExpBytes, f, 0x04010400u));     // 1152 + x
                    kh[2 * w + 1] = bitcast<half2_t>(__builtin_amdgcn_perm(kExpBytes, f, 0x04030402u));
                }
                const half2_t sc = bitcast<half2_t>(kb.sc[j]);
                const float s0 = (float)sc.x * logit_scale;
                const float s1 = (float)sc.y * logit_scale;
#pragma unroll
                for (int g = 0; g < GT; ++g) {
                    float d0 = qb[g][0], d1 = qb[g][1];
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        d0 = dot2(q[g][i], kh[i], d0);
                        d1 = dot2(q[g][4 + i], kh[4 + i], d1);
                    }
                    part[g][j] = __builtin_fmaf(d1, s1, d0 * s0);
                }
            }

            // reduce-scatter inside the quad (slot k here and slot k ^ 2 of the xor-2 partner are the
            // same token), then all-reduce across the quads of the slot: the lane ends with the complete
            // logit of token tp
            bool rescale = false;
            float m_new[GT];
#pragma unroll
            for (int g = 0; g < GT; ++g) {
                const float u0 = part[g][0] + dpp_f32<kDppXor2>(part[g][2]);
                const float u1 = part[g][1] + dpp_f32<kDppXor2>(part[g][3]);
                float logit = u0 + dpp_f32<kDppXor1>(u1);
                if (LPS >= 8) logit += dpp_f32<kDppHalfMirror>(logit);
                if (LPS >= 16) logit += dpp_f32<kDppMirror>(logit);
                if (MASK || !full) {
                    const int tk = kb.pos + tp * tpl + tsub;
                    const bool ok = tk >= pa32 && tk < pe32;
                    if (MASK && ok && g_first + g < G) {
                        const int h = kvh * G + g_first + g;
                        logit += (float)mask_row[(int64_t)h * a.mask_stride_h + tk] * kLog2e;
                    }
                    if (!ok) logit = -INFINITY;
                }
                // block max over the quad (= over the block's tokens)
                float mx = fmaxf(logit, dpp_f32<kDppXor1>(logit));
                mx = fmaxf(mx, dpp_f32<kDppXor2>(mx));
                m_new[g] = fmaxf(m_run[g], mx);
                rescale = rescale || (m_new[g] > m_run[g]);
                p[g] = __builtin_amdgcn_exp2f(logit - m_new[g]);
            }
            if (__builtin_amdgcn_ballot_w64(rescale) != 0) { // wave-uniform and rare: a running max moved
#pragma unroll
                for (int g = 0; g < GT; ++g) {
                    const float al = __builtin_amdgcn_exp2f(m_run[g] - m_new[g]);
                    m_run[g] = m_new[g];
                    l_run[g] *= al;
#pragma unroll
                    for (int c = 0; c < 16; ++c) acc[g][c] *= al;
                }
            }
#pragma unroll
            for (int g = 0; g < GT; ++g) l_run[g] += p[g];
        };

        // ---- PV of one block: int8 values converted straight to fp32 (exact), fp32 weights p * scale,
        // fp32 multiply-accumulate in the two-source form (v_fmac_f32), which issues at twice the rate
        // of the three-source and packed forms on this chip ----
        auto accumulate_pv = [&](VBlock& vb, bool fast) {
#pragma unroll
            for (int j = 0; j < kTB; ++j) {
                if (fast) {
                    if (j == 0) wait_loads<22>(vb.q8[0], vb.sc[0]);
                    if (j == 1) wait_loads<20>(vb.q8[1], vb.sc[1]);
                    if (j == 2) wait_loads<18>(vb.q8[2], vb.sc[2]);
                    if (j == 3) wait_loads<16>(vb.q8[3], vb.sc[3]);
                }
                float x[16];
#pragma unroll
                for (int w = 0; w < 4; ++w) {
                    x[4 * w + 0] = byte_to_f32<0>(vb.q8[j][w]);
                    x[4 * w + 1] = byte_to_f32<1>(vb.q8[j][w]);
                    x[4 * w + 2] = byte_to_f32<2>(vb.q8[j][w]);
                    x[4 * w + 3] = byte_to_f32<3>(vb.q8[j][w]);
                }
                const half2_t sc = bitcast<half2_t>(vb.sc[j]);
                const float sv0 = (float)sc.x, sv1 = (float)sc.y;
#pragma unroll
                for (int g = 0; g < GT; ++g) {
                    const float pj = quad_xor(p[g], j); // slot j holds token j ^ tp, whose probability is in quad lane (lane ^ j)
                    const float w0 = pj * sv0, w1 = pj * sv1;
#pragma unroll
                    for (int c = 0; c < 8; ++c) {
                        acc[g][c] = __builtin_fmaf(w0, x[c], acc[g][c]);
                        acc[g][8 + c] = __builtin_fmaf(w1, x[8 + c], acc[g][8 + c]);
                    }
                }
            }
        };

        // Wave blocks of this piece are aligned to wg_tokens in sequence coordinates, so that a block
        // never straddles a page.  At most the first and the last block of a wave are partial; they take
        // the simple path.  The full blocks in between run software-pipelined: K of block i+1 is
        // requested before the logits of block i, V of block i+1 before the PV of block i, so that three
        // half-blocks of cache bytes are in registers or in flight at any time.
        auto simple_block = [&](int pos) {
            KBlock kx;
            VBlock vx;
            issue_k(kx, pos, false);
            issue_v(vx, pos, kx.boff, false);
            logits_softmax(kx, false, false);
            accumulate_pv(vx, false);
        };
        int pos = (int)(pa / wg_tokens * wg_tokens) + wave * wave_tokens;
        if (pos + wave_tokens <= pa32) pos += wg_tokens;
        if (pos < pe32 && pos < pa32) {
            simple_block(pos);
            pos += wg_tokens;
        }
        int n_full = (pos + wave_tokens <= pe32) ? (pe32 - wave_tokens - pos) / wg_tokens + 1 : 0;
        if (kHandScheduled && n_full > 0) {
            // Every block requests the next one unconditionally (the last re-requests itself): with no
            // branch around the loads, and no register copies between stages (two named buffer pairs,
            // loop unrolled by two), the hardware wait counts stay exact.
            KBlock ka, kb;
            VBlock va, vb;
            __builtin_amdgcn_s_waitcnt(0x0F70); // vmcnt(0): the explicit wait counts below assume that only the loop's own loads are in flight
            issue_k_fast(ka, pos);
            issue_v_fast(va, ka.boff);
            // the first block has landed before the loop is entered: any register copy the compiler
            // places on the loop's entry edge then copies data, not a register still being loaded
            drain_loads(ka.q8, ka.sc);
            drain_loads(va.q8, va.sc);
            for (int i = 0;;) {
                // even block: consume (ka, va), request (kb, vb)
                int npos = pos + (i + 1 < n_full ? wg_tokens : 0);
                issue_k_fast(kb, npos);
                logits_softmax(ka, true, true);
                issue_v_fast(vb, kb.boff);
                accumulate_pv(va, true);
                pos = npos;
                if (++i == n_full) break;
                // odd block: consume (kb, vb), request (ka, va)
                npos = pos + (i + 1 < n_full ? wg_tokens : 0);
                issue_k_fast(ka, npos);
                logits_softmax(kb, true, true);
                issue_v_fast(va, ka.boff);
                accumulate_pv(vb, true);
                pos = npos;
                if (++i == n_full) break;
            }
            // drain the last (redundant) requests; all four staging buffers stay reserved until then
            drain_loads(ka.q8, ka.sc);
            drain_loads(kb.q8, kb.sc);
            drain_loads(va.q8, va.sc);
            drain_loads(vb.q8, vb.sc);
            pos += wg_tokens;
        }
        if (!kHandScheduled && n_full > 0) {
            // GT = 8 does not fit the register file without moving values to accumulation registers,
            // which is not compatible with loads that land behind the compiler's back: this variant
            // leaves load scheduling to the compiler.
            KBlock ka, kb;
            VBlock va, vb;
            issue_k(ka, pos, true);
            issue_v(va, pos, ka.boff, true);
            for (int i = 0;;) {
                int npos = pos + (i + 1 < n_full ? wg_tokens : 0);
                issue_k(kb, npos, true);
                logits_softmax(ka, true, false);
                issue_v(vb, npos, kb.boff, true);
                accumulate_pv(va, false);
                pos = npos;
                if (++i == n_full) break;
                npos = pos + (i + 1 < n_full ? wg_tokens : 0);
                issue_k(ka, npos, true);
                logits_softmax(kb, true, false);
                issue_v(va, npos, ka.boff, true);
                accumulate_pv(vb, false);
                pos = npos;
                if (++i == n_full) break;
            }
            pos += wg_tokens;
        }
        if (pos < pe32) simple_block(pos);

        // ---- merge the slots of each kv head through LDS, one query head at a time ----
        const bool whole = (pa == 0) && (pe == len);
        const int64_t piece = (int64_t)blockIdx.x + b;
        const int gslot = wave * SPW + slot;
        const int dup = NSLOT / kvhb; // slots per kv head
#pragma unroll
        for (int g = 0; g < GT; ++g) {
            // exp-sum of the slot = sum over the quad lanes' partial sums
            float lq = l_run[g] + dpp_f32<kDppXor1>(l_run[g]);
            lq += dpp_f32<kDppXor2>(lq);
            __syncthreads();
            if (lane_on) {
#pragma unroll
                for (int c = 0; c < 16; c += 4) {
                    *(f32x4*)&sm_acc[gslot * D + ch0 + c] = f32x4{acc[g][c], acc[g][c + 1], acc[g][c + 2], acc[g][c + 3]};
                }
                if (ls == 0) {
                    sm_m[gslot] = m_run[g];
                    sm_l[gslot] = lq;
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
#ifdef PMX_WG_TRACE
    if (tid == 0) {
        unsigned long long* tr = (unsigned long long*)(a.partial_ml + (int64_t)(a.ranges + a.decoding_batches) * a.num_heads * 2);
        const int64_t wg = blockIdx.x + (int64_t)gridDim.x * (blockIdx.y + (int64_t)gridDim.y * blockIdx.z);
        unsigned xcc = 0, hwid = 0;
        asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(xcc));
        asm volatile("s_getreg_b32 %0, hwreg(HW_REG_HW_ID)" : "=s"(hwid));
        tr[wg * 4 + 0] = trace_t0;
        tr[wg * 4 + 1] = wall_clock64();
        tr[wg * 4 + 2] = clock64() - trace_c0;
        tr[wg * 4 + 3] = ((unsigned long long)xcc << 32) | hwid;
    }
#endif
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
