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
//   * Inside a sequence the cuts between ranges are moved up to the next multiple
//     of the workgroup's block of tokens (or to the sequence end), so that every
//     piece starts on a block boundary and only its last block can be partial.
//   * Each slot keeps an online-softmax state per query head; slots are merged
//     through LDS at the end of a piece.  A piece that is a whole sequence is
//     written as final fp16 output; otherwise a float32 partial (normalised
//     output, running max, exp-sum) goes to the workspace and the combine kernel
//     merges the pieces of each sequence (kernel.cu:617-665 is the reference's
//     fused form of that merge).
#include <cstdlib>

#include "decode_common.h"

namespace pmxhip {

// Bytes of dynamic LDS the decode kernel needs: one slot-partial (D floats) per slot and query
// head, plus the (max, exp-sum) pair of each.
constexpr size_t decode_lds_bytes(int head_dim, int gt)
{
    const int lps = head_dim == 64 ? 4 : (head_dim == 256 ? 16 : 8);
    const int nslot = kWave / lps * kDecodeWaves;
    return (size_t)gt * nslot * (head_dim + 2) * sizeof(float);
}

// D: head dim (64, 96, 128, 256).  GT: query heads per kv head held in registers.
template <int D, int GT, bool PAGED, bool MASK>
__global__ __launch_bounds__(kDecodeThreads, (GT <= 4 ? 2 : 1)) void decode_attention_kernel(const DecodeLaunch a)
{
    constexpr int LPS = (D == 64) ? 4 : (D == 256 ? 16 : 8); // lanes per slot
    constexpr int LPS_ACTIVE = D / 16;                        // 6 of 8 for D = 96
    constexpr int SPW = kWave / LPS;                          // slots per wave
    constexpr int NSLOT = SPW * kDecodeWaves;
    // Inline-assembly loads with explicit wait counts in the pipelined loop.  Not for GT = 8 (does not fit
    // the register file without spills) nor with a mask (its loads are the compiler's): a spill or a
    // compiler-scheduled load inside the loop is not compatible with loads that land behind the compiler's back.
    constexpr bool kHandScheduled = GT <= 4 && !MASK;

    extern __shared__ float sm_dyn[];
    float* const sm_acc = sm_dyn;                 // [GT][NSLOT][D]
    float* const sm_m = sm_dyn + GT * NSLOT * D;  // [GT][NSLOT]
    float* const sm_l = sm_m + GT * NSLOT;        // [GT][NSLOT]

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

    // slots over (kv head, token sub-index): kv heads first.  kvhb and tpl are powers of two.
    const int kvhb = a.kv_heads_per_group;        // <= SPW
    const int kvhb_shift = __builtin_ctz(kvhb);
    const int tpl = SPW >> kvhb_shift;            // tokens one wave load covers
    const int tpl_shift = __builtin_ctz(tpl);
    const int head_local = slot & (kvhb - 1);
    const int tsub = slot >> kvhb_shift;
    const int wave_tokens = kTB * tpl;            // tokens a wave handles per iteration
    const int wg_tokens = wave_tokens * kDecodeWaves;
    const int wg_shift = __builtin_ctz(wg_tokens);

    const int kvh = blockIdx.y * kvhb + head_local;
    const int g_first = blockIdx.z * GT; // first query head (within the kv head's group) of this pass
    const int G = (int)a.num_kv_repeats;

    const const_i64_ptr kvstarts = as_constant(a.kvstarts);
    const const_i64_ptr cachestarts = as_constant(a.cachestarts);
    const int64_t kv_base = kvstarts[0];
    const int64_t total = stream_length(kvstarts[a.decoding_batches] - kv_base, a.decoding_batches);
    const int64_t per = tokens_per_range(total, a.ranges, wg_tokens, a.min_tokens_per_range);
    const int64_t r0 = (int64_t)blockIdx.x * per;
    if (r0 >= total) return;
    const int64_t r1 = (r0 + per < total) ? r0 + per : total;

    // Addressing: a wave-uniform 64-bit base per block (scalar registers) plus a 32-bit per-lane
    // offset: (token in block) * stride_s + (head in group) * stride_h + channel.
    const int64_t group_off = a.layer_idx * a.cache_stride_l + (int64_t)(blockIdx.y * kvhb) * a.cache_stride_h;
    const uint32_t stride_s32 = (uint32_t)a.cache_stride_s; // the host checks that a block's span fits 32 bits
    const uint32_t lane_base = (uint32_t)((int64_t)head_local * a.cache_stride_h + ch0);
    const char* const cache_k = (const char*)a.cache + group_off;
    const char* const cache_v = cache_k + a.cache_stride_kv;
    const char* const scale_k = (const char*)a.scale + (group_off >> 3) * 2;
    const char* const scale_v = scale_k + (a.cache_stride_kv >> 3) * 2;
    const float logit_scale = a.attn_scale * kLog2e;

    // The index entries of a sequence are read one sequence ahead (the first one's come out of the search): a piece
    // that follows another in the range starts at its sequence's first token, so kvstarts and the first page table
    // entry (contiguous cache: the sequence's first row) are known when the piece before it begins.
    int64_t seq_start, seq_end, ahead_end = 0, ahead_row = 0, first_row = 0;
    bool have_first_row = false;
    int b = find_sequence(kvstarts, a.kvstarts, (int)a.decoding_batches, r0, (int)(threadIdx.x & 63), seq_start, seq_end);
    for (; b < a.decoding_batches; ++b, seq_start = seq_end, seq_end = ahead_end, first_row = ahead_row, have_first_row = true) {
        const int64_t first_token = seq_start - kv_base;
        if (stream_length(first_token, b) >= r1) break; // the sequence's interval starts beyond the range
        const int64_t len = seq_end - seq_start;
        {
            const int64_t nb1 = b + 1 < a.decoding_batches ? b + 1 : b;
            ahead_end = kvstarts[nb1 + 1];
            ahead_row = cachestarts[PAGED ? nb1 * a.cachestarts_stride_b : nb1];
        }
        const int64_t s_beg = sequence_origin(first_token, b);
        int64_t pa, pe; // this workgroup's piece [pa, pe) of the sequence, in sequence coordinates
        piece_bounds(r0, r1, s_beg, len, wg_tokens, pa, pe);
        if (pe <= pa) continue;
        // sequence-relative positions fit 32 bits
        const int pa32 = (int)pa, pe32 = (int)pe;

        // Wave blocks: pa is a multiple of wg_tokens, so every block lies inside one page and only
        // the last block of a wave can reach beyond the piece.
        const int pos0 = pa32 + wave * wave_tokens;
        const int nb = pos0 < pe32 ? (pe32 - pos0 + wg_tokens - 1) >> wg_shift : 0;
        const bool tail_partial = nb > 0 && pos0 + ((nb - 1) << wg_shift) + wave_tokens > pe32;

        const int64_t table_base = PAGED ? (int64_t)b * a.cachestarts_stride_b : (int64_t)b;
        const int64_t seq_row0 = PAGED ? 0 : (have_first_row ? first_row : cachestarts[b]);
        const half_t* mask_row = nullptr;
        if (MASK) mask_row = (const half_t*)a.attn_mask + (int64_t)b * a.mask_stride_s + seq_start;
        const int last_page = (pe32 - 1) >> 7;

        // Page table entries are read one page ahead with scalar loads, so that no block waits
        // for its row base: `page_row` belongs to page `page_idx`, `next_row` to the page after it.
        int page_idx = have_first_row ? -1 : -2; // the row of page 0 read ahead stands in as the "next page" of page -1
        int64_t page_row = 0, next_row = first_row;
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

        // Per-lane offsets of the block being requested: those of a full block until the wave's last
        // block is requested; if that one reaches beyond the piece, its out-of-piece tokens are
        // redirected to the piece's last token (the load is harmless, the logit is masked).
        uint32_t vo[kTB], vo_sc[kTB];
#pragma unroll
        for (int j = 0; j < kTB; ++j) {
            vo[j] = (uint32_t)((j ^ tp) * tpl + tsub) * stride_s32 + lane_base;
            vo_sc[j] = vo[j] >> 2; // the same offset in the scale tensor: one fp16 scale per 8 channels
        }
        auto clamp_offsets = [&](int pos) {
#pragma unroll
            for (int j = 0; j < kTB; ++j) {
                const int t = pos + (j ^ tp) * tpl + tsub;
                const int tc = t < pe32 ? t : pe32 - 1;
                vo[j] = (uint32_t)(tc - pos) * stride_s32 + lane_base;
                vo_sc[j] = vo[j] >> 2;
            }
        };

        // ---- requests of one wave block (positions pos .. pos + wave_tokens): K with its scales, V with
        // its scales, in a fixed order (token 0: 16 bytes then scales, token 1: ..., 8 operations per
        // half-block) ----
        auto request_k = [&](KBlock& kb, int pos) {
            kb.pos = pos;
            const int64_t boff = row_base_of(pos) * a.cache_stride_s;
            kb.boff = boff;
            const char* bk = cache_k + boff;
            const char* sk = scale_k + (boff >> 3) * 2;
#pragma unroll
            for (int j = 0; j < kTB; ++j) {
                if (kHandScheduled) {
                    load_b128<false>(kb.q8[j], vo[j], bk);
                    load_b32<false>(kb.sc[j], vo_sc[j], sk);
                } else {
                    kb.q8[j] = *(const u32x4*)(bk + vo[j]);
                    kb.sc[j] = *(const uint32_t*)(sk + vo_sc[j]);
                }
            }
        };
        auto request_v = [&](VBlock& vb, int64_t boff) {
            const char* bv = cache_v + boff;
            const char* sv = scale_v + (boff >> 3) * 2;
#pragma unroll
            for (int j = 0; j < kTB; ++j) {
                if (kHandScheduled) {
                    load_b128<false>(vb.q8[j], vo[j], bv);
                    load_b32<false>(vb.sc[j], vo_sc[j], sv);
                } else {
                    vb.q8[j] = *(const u32x4*)(bv + vo[j]);
                    vb.sc[j] = *(const uint32_t*)(sv + vo_sc[j]);
                }
            }
        };

        // The first block is requested before anything else of the piece, so that its latency overlaps
        // the query loads below.
        KBlock ka, kb;
        VBlock va, vb;
        int pos = pos0;
        if (nb > 0) {
            if (nb == 1 && tail_partial) clamp_offsets(pos);
            request_k(ka, pos);
            request_v(va, ka.boff);
        }

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

        // ---- QK^T and softmax of one block: leaves this lane's probability (token tp) in p[g] ----
        float p[GT];
        auto logits_softmax = [&](KBlock& kb) {
            // logits, still partial over the slot's lanes: part[g][j], log2 units
            float part[GT][kTB];
#pragma unroll
            for (int j = 0; j < kTB; ++j) {
                if (kHandScheduled) {
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
                    float d0 = dot2_init(q[g][0], kh[0], qb[g][0]);
                    float d1 = dot2_init(q[g][4], kh[4], qb[g][1]);
#pragma unroll
                    for (int i = 1; i < 4; ++i) {
                        d0 = dot2(q[g][i], kh[i], d0);
                        d1 = dot2(q[g][4 + i], kh[4 + i], d1);
                    }
                    part[g][j] = __builtin_fmaf(d1, s1, d0 * s0);
                }
            }

            // reduce-scatter inside the quad (slot k here and slot k ^ 2 of the xor-2 partner are the
            // same token), then all-reduce across the quads of the slot: the lane ends with the complete
            // logit of token tp
            const int tk = kb.pos + tp * tpl + tsub;
            const bool ok = tk < pe32; // false only in a wave's last block, for tokens beyond the piece
            bool rescale = false;
            float m_new[GT];
#pragma unroll
            for (int g = 0; g < GT; ++g) {
                const float u0 = part[g][0] + dpp_f32<kDppXor2>(part[g][2]);
                const float u1 = part[g][1] + dpp_f32<kDppXor2>(part[g][3]);
                float logit = u0 + dpp_f32<kDppXor1>(u1);
                if (LPS >= 8) logit += dpp_f32<kDppHalfMirror>(logit);
                if (LPS >= 16) logit += dpp_f32<kDppMirror>(logit);
                if (MASK && ok && g_first + g < G) {
                    const int h = kvh * G + g_first + g;
                    logit += (float)mask_row[(int64_t)h * a.mask_stride_h + tk] * kLog2e;
                }
                logit = ok ? logit : -INFINITY;
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
        auto accumulate_pv = [&](VBlock& vb) {
#pragma unroll
            for (int j = 0; j < kTB; ++j) {
                if (kHandScheduled) {
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

        // The blocks run software-pipelined: K of block i+1 is requested before the logits of block i,
        // V of block i+1 before the PV of block i, so that three half-blocks of cache bytes are in
        // registers or in flight at any time.  Every block requests the next one unconditionally (the
        // last re-requests itself): with no branch around the loads, and no register copies between
        // stages (two named buffer pairs, loop unrolled by two), the hardware wait counts stay exact.
        if (nb > 0) {
            if (kHandScheduled) {
                // The first block has landed before the loop is entered, and nothing else is in flight:
                // the wait counts of the loop count the loop's own requests only, and any register copy
                // the compiler places on the loop's entry edge copies data, not a register being loaded.
                drain_loads(ka.q8, ka.sc);
                drain_loads(va.q8, va.sc);
            }
            for (int i = 0;;) {
                // even block: consume (ka, va), request (kb, vb)
                int npos = pos + (i + 1 < nb ? wg_tokens : 0);
                if (tail_partial && i + 2 == nb) clamp_offsets(npos);
                request_k(kb, npos);
                logits_softmax(ka);
                request_v(vb, kb.boff);
                accumulate_pv(va);
                pos = npos;
                if (++i == nb) break;
                // odd block: consume (kb, vb), request (ka, va)
                npos = pos + (i + 1 < nb ? wg_tokens : 0);
                if (tail_partial && i + 2 == nb) clamp_offsets(npos);
                request_k(ka, npos);
                logits_softmax(kb);
                request_v(va, ka.boff);
                accumulate_pv(vb);
                pos = npos;
                if (++i == nb) break;
            }
            if (kHandScheduled) {
                // drain the last (redundant) requests; all four staging buffers stay reserved until then
                drain_loads(ka.q8, ka.sc);
                drain_loads(kb.q8, kb.sc);
                drain_loads(va.q8, va.sc);
                drain_loads(vb.q8, vb.sc);
            }
        }

        // ---- merge the slots of each kv head through LDS, all query heads in one pass ----
        const bool whole = (pa == 0) && (pe == len);
        const int64_t piece = (int64_t)blockIdx.x + b;
        const int gslot = wave * SPW + slot;
        const int dup = NSLOT >> kvhb_shift; // slots per kv head
#pragma unroll
        for (int g = 0; g < GT; ++g) {
            // exp-sum of the slot = sum over the quad lanes' partial sums
            float lq = l_run[g] + dpp_f32<kDppXor1>(l_run[g]);
            lq += dpp_f32<kDppXor2>(lq);
            if (lane_on) {
                float* dst = sm_acc + (g * NSLOT + gslot) * D + ch0;
#pragma unroll
                for (int c = 0; c < 16; c += 4) *(f32x4*)(dst + c) = f32x4{acc[g][c], acc[g][c + 1], acc[g][c + 2], acc[g][c + 3]};
                if (ls == 0) {
                    sm_m[g * NSLOT + gslot] = m_run[g];
                    sm_l[g * NSLOT + gslot] = lq;
                }
            }
        }
        __syncthreads();
        // one output quad (4 channels of one (query head, kv head)) per thread and step
        constexpr int QPH = D / 4; // quads per head
        for (int idx = tid; idx < GT * kvhb * QPH; idx += kDecodeThreads) {
            const int c = (idx % QPH) * 4;
            const int gh = idx / QPH;
            const int hl = gh & (kvhb - 1);
            const int g = gh >> kvhb_shift;
            const int gi = g_first + g;
            if (gi >= G) continue;
            // slots of kv head hl: slot hl + kvhb * (k % tpl) of wave k / tpl
            float M = kNegBig;
            for (int k = 0; k < dup; ++k) {
                const int sidx = (k >> tpl_shift) * SPW + hl + ((k & (tpl - 1)) << kvhb_shift);
                M = fmaxf(M, sm_m[g * NSLOT + sidx]);
            }
            float L = 0.f;
            f32x4 O = {0.f, 0.f, 0.f, 0.f};
            for (int k = 0; k < dup; ++k) {
                const int sidx = (k >> tpl_shift) * SPW + hl + ((k & (tpl - 1)) << kvhb_shift);
                const float w = __builtin_amdgcn_exp2f(sm_m[g * NSLOT + sidx] - M);
                L += sm_l[g * NSLOT + sidx] * w;
                const f32x4 v = *(const f32x4*)(sm_acc + (g * NSLOT + sidx) * D + c);
                O += v * w;
            }
            const float inv = L > 0.f ? 1.f / L : 0.f;
            O *= inv;
            const int h = (blockIdx.y * kvhb + hl) * G + gi;
            if (whole) {
                half_t* out = (half_t*)a.output + (int64_t)b * a.output_stride_s + (int64_t)h * D + c;
                typedef half_t half4_t __attribute__((ext_vector_type(4)));
                *(half4_t*)out = half4_t{(half_t)O[0], (half_t)O[1], (half_t)O[2], (half_t)O[3]};
            } else {
                *(f32x4*)(a.partial_out + (piece * a.num_heads + h) * D + c) = O;
                if (c == 0) {
                    a.partial_ml[(piece * a.num_heads + h) * 2 + 0] = M;
                    a.partial_ml[(piece * a.num_heads + h) * 2 + 1] = L;
                }
            }
        }
        __syncthreads(); // the next piece overwrites the LDS partials
    }
}

// One workgroup of NW waves per (sequence, query head): merges the pieces the decode kernel left in the
// workspace.  A sequence with a single piece was already written by the decode kernel.  The (max, exp-sum)
// pairs are read with lanes over ranges (every wave for itself, so no exchange is needed for the maximum
// and the denominator); the rows are read four channels per lane, so a wave takes 64 / (D/4) pieces per
// request and keeps four requests in flight, and the waves share the pieces of a long sequence between
// them.  Their partial rows are added through LDS.
template <int D, int NW>
__global__ __launch_bounds__(64 * NW) void decode_combine_kernel(const DecodeLaunch a)
{
    constexpr int LPR = D / 4;    // lanes that cover one piece row
    constexpr int PPW = 64 / LPR; // piece rows per wave and request (D = 96: two, the last 16 lanes idle)
    constexpr int SLOTS = NW * PPW;
    constexpr int U = 4;
    __shared__ float s_part[SLOTS][D];
    const int b = blockIdx.y;
    const int h = blockIdx.x;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int sub = lane / LPR, c4 = lane % LPR;
    const int slot = (tid >> 6) * PPW + sub;
    const int64_t kv_base = a.kvstarts[0];
    const int64_t total = stream_length(a.kvstarts[a.decoding_batches] - kv_base, a.decoding_batches);
    const int64_t s_beg = sequence_origin(a.kvstarts[b] - kv_base, b);
    const int64_t s_end = s_beg + (a.kvstarts[b + 1] - a.kvstarts[b]);
    int64_t out_row = b;
    int out_head = h;
    if (a.seqstarts != nullptr) { // chunks of query tokens: h is a (query position, query head) column of a kv head
        const int gv = (int)a.num_kv_repeats, gr = a.chunk_q_heads;
        const int gq = h % gv, cpos = gq / gr;
        out_row = a.seqstarts[b];
        const int64_t chunk_rows = a.seqstarts[b + 1] - out_row;
        if (h == 0 && chunk_rows > gv / gr) {
            // The caller's max_seqlen is smaller than this sequence's chunk: the step has no column for the rows
            // beyond it.  They are filled with NaN rather than left as they were, so that the understated hint shows.
            const int64_t row_halves = (a.num_heads / gv) * gr * D; // query heads * head_dim
            for (int64_t r = gv / gr; r < chunk_rows; ++r) {
                half_t* row = (half_t*)a.output + (out_row + r) * a.output_stride_s;
                for (int64_t c = tid; c < row_halves; c += 64 * NW) row[c] = bitcast<half_t>((uint16_t)0x7E00);
            }
        }
        if (cpos >= (int)chunk_rows) return; // the sequence's chunk is shorter
        out_row += cpos;
        out_head = (h / gv) * gr + (gq - cpos * gr);
    }
    half_t* out = (half_t*)a.output + out_row * a.output_stride_s + (int64_t)out_head * D;
    if (s_end <= s_beg) { // empty sequence: the reference yields 0/(0+1e-6) = 0 (kernel.cu:516)
        for (int c = tid; c < D; c += 64 * NW) out[c] = (half_t)0.f;
        return;
    }
    const int64_t per = tokens_per_range(total, a.ranges, a.wg_tokens, a.min_tokens_per_range);
    const int64_t w0 = s_beg / per, w1 = (s_end - 1) / per;
    if (w0 == w1) return; // one range covers the sequence: final output already written

    f32x4 o = {0.f, 0.f, 0.f, 0.f};
    float den = 0.f;
    if (w1 - w0 < 64) {
        // at most 64 ranges (one per lane): the first rows are requested together with the (max, sum) pairs,
        // before their weights are known, so that the two round trips to memory overlap
        const int n = (int)(w1 - w0) + 1;
        f32x4 row[U];
        int src[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int k = u * SLOTS + slot;
            const bool mine = k < n && sub < PPW;
            src[u] = mine ? k : -1;
            row[u] = *(const f32x4*)(a.partial_out + ((w0 + (mine ? k : n - 1) + b) * a.num_heads + h) * D + c4 * 4);
        }
        float m = kNegBig, l = 0.f;
        bool live = false;
        if (lane < n) {
            const int64_t w = w0 + lane;
            int64_t pa, pe;
            const int64_t r0 = w * per;
            piece_bounds(r0, (r0 + per < total) ? r0 + per : total, s_beg, s_end - s_beg, a.wg_tokens, pa, pe);
            live = pe > pa;
            if (live) {
                const float2 ml = *(const float2*)(a.partial_ml + ((w + b) * a.num_heads + h) * 2);
                m = ml.x;
                l = ml.y;
            }
        }
        if (__builtin_popcountll(__builtin_amdgcn_ballot_w64(live)) <= 1) return; // the decode kernel wrote the final output
        float M = m;
#pragma unroll
        for (int s = 32; s >= 1; s >>= 1) M = fmaxf(M, __shfl_xor(M, s));
        const float wt = live ? l * __builtin_amdgcn_exp2f(m - M) : 0.f; // an empty piece's row may be stale: weight zero
        den = wt;
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const float wk = __shfl(wt, src[u] < 0 ? 0 : src[u]);
            if (src[u] >= 0 && wk != 0.f) o += row[u] * wk;
        }
        for (int k0 = SLOTS * U; k0 < n; k0 += SLOTS * U) {
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int k = k0 + u * SLOTS + slot;
                const bool mine = k < n && sub < PPW;
                src[u] = mine ? k : -1;
                row[u] = *(const f32x4*)(a.partial_out + ((w0 + (mine ? k : n - 1) + b) * a.num_heads + h) * D + c4 * 4);
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const float wk = __shfl(wt, src[u] < 0 ? 0 : src[u]);
                if (src[u] >= 0 && wk != 0.f) o += row[u] * wk;
            }
        }
    } else {
        // lanes over ranges: the maximum over the non-empty pieces
        float M = kNegBig;
        int pieces = 0;
        for (int64_t wb = w0; wb <= w1; wb += 64) {
            const int64_t w = wb + lane;
            float m = kNegBig;
            bool live = false;
            if (w <= w1) {
                int64_t pa, pe;
                const int64_t r0 = w * per;
                piece_bounds(r0, (r0 + per < total) ? r0 + per : total, s_beg, s_end - s_beg, a.wg_tokens, pa, pe);
                live = pe > pa;
                if (live) m = a.partial_ml[((w + b) * a.num_heads + h) * 2];
            }
            pieces += __builtin_popcountll(__builtin_amdgcn_ballot_w64(live));
            M = fmaxf(M, m);
        }
        if (pieces <= 1) return; // the cuts moved onto one boundary: the decode kernel wrote the final output
#pragma unroll
        for (int s = 32; s >= 1; s >>= 1) M = fmaxf(M, __shfl_xor(M, s));

        for (int64_t wb = w0; wb <= w1; wb += 64) {
            const int64_t w = wb + lane;
            float wt = 0.f; // weight of range wb + lane
            if (w <= w1) {
                int64_t pa, pe;
                const int64_t r0 = w * per;
                piece_bounds(r0, (r0 + per < total) ? r0 + per : total, s_beg, s_end - s_beg, a.wg_tokens, pa, pe);
                if (pe > pa) {
                    const int64_t pi = (w + b) * a.num_heads + h;
                    wt = a.partial_ml[pi * 2 + 1] * __builtin_amdgcn_exp2f(a.partial_ml[pi * 2] - M);
                }
            }
            den += wt;
            const int n = (int)((w1 - wb < 63 ? w1 - wb : 63) + 1);
            // U requests per slot in flight; an empty piece has weight zero and a possibly stale workspace row,
            // which is read but never enters the sum
            for (int k0 = 0; k0 < n; k0 += SLOTS * U) {
                float wk[U];
                f32x4 row[U];
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    const int k = k0 + u * SLOTS + slot;
                    const bool mine = k < n && sub < PPW;
                    const int kc = mine ? k : n - 1;
                    wk[u] = __shfl(wt, kc);
                    if (!mine) wk[u] = 0.f;
                    row[u] = *(const f32x4*)(a.partial_out + ((wb + kc + b) * a.num_heads + h) * D + c4 * 4);
                }
#pragma unroll
                for (int u = 0; u < U; ++u)
                    if (wk[u] != 0.f) o += row[u] * wk[u];
            }
        }
    }
#pragma unroll
    for (int s = 32; s >= 1; s >>= 1) den += __shfl_xor(den, s);
    if (sub < PPW) *(f32x4*)&s_part[slot][c4 * 4] = o;
    __syncthreads();
    if (tid < LPR) {
        f32x4 r = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int i = 0; i < SLOTS; ++i) r += *(const f32x4*)&s_part[i][tid * 4];
        const float inv = den > 0.f ? 1.f / den : 0.f;
        r *= inv;
        typedef half_t half4_t __attribute__((ext_vector_type(4)));
        *(half4_t*)(out + tid * 4) = half4_t{(half_t)r[0], (half_t)r[1], (half_t)r[2], (half_t)r[3]};
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

template <int D, int GT, bool PAGED, bool MASK>
static DeviceMask& decode_variant_ready()
{
    static DeviceMask ready{0};
    return ready;
}

template <int D, int GT, bool PAGED, bool MASK>
static int launch_decode_variant(const DecodeLaunch& a, dim3 grid, hipStream_t stream)
{
    constexpr size_t lds_bytes = decode_lds_bytes(D, GT);
    // above the default limit of dynamic LDS per workgroup for the wider variants
    if (int rc = ensure_dynamic_lds((const void*)decode_attention_kernel<D, GT, PAGED, MASK>, (int)lds_bytes, stream,
                                    decode_variant_ready<D, GT, PAGED, MASK>()))
        return rc;
    hipLaunchKernelGGL((decode_attention_kernel<D, GT, PAGED, MASK>), grid, dim3(kDecodeThreads), lds_bytes, stream, a);
    return kLaunchOk;
}

template <int D, int GT>
static int launch_decode_dgt(const DecodeLaunch& a, dim3 grid, hipStream_t stream)
{
    const bool paged = a.cache_mode == 1;
    const bool mask = a.attn_mask != nullptr;
    if (paged) return mask ? launch_decode_variant<D, GT, true, true>(a, grid, stream)
                           : launch_decode_variant<D, GT, true, false>(a, grid, stream);
    return mask ? launch_decode_variant<D, GT, false, true>(a, grid, stream)
                : launch_decode_variant<D, GT, false, false>(a, grid, stream);
}

template <int D>
static int launch_decode_d(const DecodeLaunch& a, int stage, hipStream_t stream)
{
    if (stage != 2) {
        switch (a.kernel) {
            case kDecodeKernelMfma16:
            case kDecodeKernelMfma32:
                if (D != 128 && !(D == 64 && a.kernel == kDecodeKernelMfma32)) return kLaunchNoKernel;
                launch_decode_mfma(a, stream);
                break;
            case kDecodeKernelQuad:
                if (D != 64 && D != 128 && D != 256) return kLaunchNoKernel;
                launch_decode_quad(a, stream);
                break;
            case kDecodeKernelGeneral: {
                const dim3 grid((unsigned)a.ranges, (unsigned)(a.num_kv_heads / a.kv_heads_per_group), (unsigned)a.num_passes);
                int rc = kLaunchNoKernel;
                switch (a.q_heads_per_pass) {
                    case 1: rc = launch_decode_dgt<D, 1>(a, grid, stream); break;
                    case 2: rc = launch_decode_dgt<D, 2>(a, grid, stream); break;
                    case 4: rc = launch_decode_dgt<D, 4>(a, grid, stream); break;
                    case 8: rc = launch_decode_dgt<D, 8>(a, grid, stream); break;
                    default: break;
                }
                if (rc != kLaunchOk) return rc;
                break;
            }
            default: return kLaunchNoKernel;
        }
    }
    if (stage == 1) return kLaunchOk;
    // always run: it also writes the zero rows of empty sequences
    {
        // waves per (sequence, head) row by the mean number of pieces per sequence: with many rows of a few
        // pieces each, extra waves only add dispatch work (measured: 8 / 9 / 13 us for 1 / 2 / 4 waves on 128
        // sequences of about five pieces, 17 / 12 / 9 us on one sequence of 256 pieces)
        const dim3 cgrid((unsigned)a.num_heads, (unsigned)a.decoding_batches);
        if (a.ranges <= 16 * a.decoding_batches) hipLaunchKernelGGL((decode_combine_kernel<D, 1>), cgrid, dim3(64), 0, stream, a);
        else if (a.ranges <= 48 * a.decoding_batches) hipLaunchKernelGGL((decode_combine_kernel<D, 2>), cgrid, dim3(128), 0, stream, a);
        else hipLaunchKernelGGL((decode_combine_kernel<D, 4>), cgrid, dim3(256), 0, stream, a);
    }
    return kLaunchOk;
}

// the one-time attribute call of every variant (pmxhip_init)
template <int D, int GT>
static int init_decode_dgt()
{
    int rc = kLaunchOk;
    auto one = [&](const void* k, DeviceMask& ready) {
        if (rc == kLaunchOk) rc = set_dynamic_lds_once(k, (int)decode_lds_bytes(D, GT), ready);
    };
    one((const void*)decode_attention_kernel<D, GT, true, true>, decode_variant_ready<D, GT, true, true>());
    one((const void*)decode_attention_kernel<D, GT, true, false>, decode_variant_ready<D, GT, true, false>());
    one((const void*)decode_attention_kernel<D, GT, false, true>, decode_variant_ready<D, GT, false, true>());
    one((const void*)decode_attention_kernel<D, GT, false, false>, decode_variant_ready<D, GT, false, false>());
    return rc;
}
template <int D>
static int init_decode_d()
{
    if (int rc = init_decode_dgt<D, 1>()) return rc;
    if (int rc = init_decode_dgt<D, 2>()) return rc;
    if (int rc = init_decode_dgt<D, 4>()) return rc;
    return init_decode_dgt<D, 8>();
}
int init_decode_kernels()
{
    if (int rc = init_decode_d<64>()) return rc;
    if (int rc = init_decode_d<96>()) return rc;
    if (int rc = init_decode_d<128>()) return rc;
    return init_decode_d<256>();
}

int launch_decode(const DecodeLaunch& a, int stage, hipStream_t stream)
{
    switch (a.head_dim) {
        case 64: return launch_decode_d<64>(a, stage, stream);
        case 96: return launch_decode_d<96>(a, stage, stream);
        case 128: return launch_decode_d<128>(a, stage, stream);
        case 256: return launch_decode_d<256>(a, stage, stream);
        default: return kLaunchNoKernel;
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
