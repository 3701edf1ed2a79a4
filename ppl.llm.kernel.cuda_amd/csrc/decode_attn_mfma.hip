// Decode attention over the int8 group-8 KV cache, variant for five and more query heads per kv head at
// head_dim 128 or 64 (reference: src/ppl/kernel/llm/cuda/pmx/multi_head_cache_attention/kernel.cu:1090-1891,
// the GQCA kernel, which also puts the query heads of a kv head on tensor cores).
//
// With that many query heads the per-head arithmetic of the VALU kernels outweighs the cache stream.
// Here a wave owns one kv head and treats its query heads as the columns of a small matrix product:
//   S^T = K Q^T   (32 tokens x 32 columns, v_mfma_f32_32x32x16_f16, K from registers)
//   O^T = V^T P^T (128 channels x 32 columns, V^T from a wave-private LDS tile)
// so the arithmetic per cache byte no longer grows with the number of query heads; what stays on the
// VALU is the dequantisation (once per byte) and a softmax over 32 x 32 logits per block.
//
// Two variants: up to sixteen query heads per kv head at head_dim 128 use v_mfma_f32_16x16x32_f16 (half the columns,
// half the MFMA time, half the logits per lane); the 32x32x16 form serves seventeen and more, and head_dim 64.  More
// than 32 query heads per kv head (multi-query models: 48 or 71 query heads on one kv head) run as passes of 32
// columns (blockIdx.z), each of which reads the cache again: the bytes of one kv head are few and stay in the L2.
//
// Exactness follows the prefill kernel: K^ = int8 * scale, V^ and p are kept as hi + lo pairs of halves
// (2 MFMAs per QK step, 3 per PV step), so no fp16 rounding of the dequantised cache enters the result.
//
// Ranges, pieces and the workspace are those of decode_attn.hip: one workgroup (a wave per kv head: four, or two
// or one when the kv heads do not come in fours) per token range, cuts on multiples of 32 tokens, float32 pieces merged by decode_combine_kernel.
#include <cstdlib>

#include "decode_common.h"

namespace pmxhip {

namespace {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int kMfmaD = 128;
constexpr int kMfmaBlock = 32;  // tokens per wave iteration (rows of one MFMA block)
constexpr float kPShift = 14.0f; // p is kept as 2^14 * exp2(logit - max): its half parts stay normal numbers

// position of token offset o (0..15) inside its 16-token group of the transposed V tile:
// token bits (a, h, r1, r0) -> position bits (h, a, r1, r0), the order in which a lane of the
// S^T accumulator holds its tokens
__device__ __forceinline__ int vt_pos16(int o) { return ((o & 4) << 1) | ((o & 8) >> 1) | (o & 3); }

// V^T tile of one wave: 128 channel rows of 32 halves (64 bytes = four 16-byte blocks).  The transposing
// stores of one instruction come from 64 lanes whose rows are 8 apart (a multiple of the bank cycle), so
// (a) channel e of group g lives in row 8 g + (e & 4) + ((e + g) & 3): the rows of one instruction then
// cover all four 64-byte bank windows, and (b) the block index is XORed with bits 2..3 and 5..6 of the
// row, which spreads them over the four blocks of a window and keeps the 16-byte fragment reads of eight
// consecutive rows on different banks without padding.
__device__ __forceinline__ int vt_row(int channel)
{
    const int g = channel >> 3;
    return (channel & ~3) | ((channel + g) & 3);
}
__device__ __forceinline__ int vt_index(int row /* from vt_row */, int pos /* 0..31, multiple of 4 or 8 */)
{
    return row * 32 + ((((pos >> 3) ^ (row >> 2) ^ (row >> 5)) & 3) << 3) + (pos & 7);
}

} // namespace

// D: head_dim 128 or 64 (half the k-steps, channel blocks and V units).  blockIdx.z: which 32 query heads of the
// kv head's group are this launch's columns (more than 32 query heads per kv head take several passes over the cache).
// CHUNK: the sequences have a few query tokens each instead of one (short prefill chunks, the candidate tokens of
// speculative decoding: a.seqstarts gives their query rows).  The columns of a kv head are then (query position,
// query head) pairs, column = position * (query heads per kv head) + head, a.num_kv_repeats counts those columns and
// a.num_heads the columns of all kv heads; a column attends the tokens below its own causal limit.  Everything else
// -- ranges, pieces, workspace -- is the decode step's, with columns in place of query heads.
template <int NW, bool PAGED, bool MASK, int D, bool CHUNK = false>
__global__ __launch_bounds__(NW * kWave, 2) void decode_attention_mfma_kernel(const DecodeLaunch a)
{
    static_assert(D == 128 || D == 64, "head_dim");
    static_assert(!(CHUNK && MASK), "no attn_mask form for chunks");
    constexpr int HALF = D / 2; // channels of a token that a half-wave's lanes hold as K bytes
    constexpr int KW = D / 32;  // 16-byte words of those bytes
    constexpr int KS = D / 16;  // k-steps of S^T
    constexpr int CB = D / 32;  // 32-channel blocks of O^T
    constexpr int GPT = D / 8;  // quantisation groups per token
    constexpr int VU = D / 64;  // (token quad, group) units of V per lane
    __shared__ __attribute__((aligned(16))) half_t s_vt[NW][2][D * kMfmaBlock]; // [wave][hi, lo]

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31; // token row (K operand), channel row (V operand) or column (query head)
    const int hh = lane >> 5;
    const int G = (int)a.num_kv_repeats;
    const int gq = blockIdx.z * kMfmaBlock + l32; // this lane's column: query head gq of the kv head's group
    const int GR = CHUNK ? (int)a.chunk_q_heads : G;       // query heads per kv head
    const int cpos = CHUNK ? gq / GR : 0;                  // the column's query position within its sequence's chunk
    const int cg = CHUNK ? gq - cpos * GR : gq;            // ... and its query head within the kv head's group
    const int kvh = blockIdx.y * NW + wave;
    half_t* const sV = s_vt[wave][0];
    half_t* const sVlo = s_vt[wave][1];

    const const_i64_ptr kvstarts = as_constant(a.kvstarts);
    const const_i64_ptr cachestarts = as_constant(a.cachestarts);
    const int64_t kv_base = kvstarts[0];
    const int64_t total = stream_length(kvstarts[a.decoding_batches] - kv_base, a.decoding_batches);
    const int64_t per = tokens_per_range(total, a.ranges, kMfmaBlock, a.min_tokens_per_range);
    const int64_t r0 = (int64_t)blockIdx.x * per;
    if (r0 >= total) return;
    const int64_t r1 = (r0 + per < total) ? r0 + per : total;

    const int64_t head_off = a.layer_idx * a.cache_stride_l + (int64_t)kvh * a.cache_stride_h;
    const uint32_t stride_s32 = (uint32_t)a.cache_stride_s; // the host checks that a block's span fits 32 bits
    const char* const cache_k = (const char*)a.cache + head_off;
    const char* const cache_v = cache_k + a.cache_stride_kv;
    const half_t* const scale_k = (const half_t*)a.scale + (head_off >> 3);
    const half_t* const scale_v = scale_k + (a.cache_stride_kv >> 3);
    const float sm_scale = a.attn_scale * kLog2e;

    // V units of this lane: (token quad, channel group) pairs idx = lane + 64 u, group = idx % GPT, quad = idx / GPT
    const int v_g = lane % GPT;
    int v_q[VU];
#pragma unroll
    for (int u = 0; u < VU; ++u) v_q[u] = (lane + 64 * u) / GPT;

    int b = find_sequence(kvstarts, a.kvstarts, (int)a.decoding_batches, r0, lane);
    for (; b < a.decoding_batches; ++b) {
        const int64_t first_token = kvstarts[b] - kv_base;
        if (stream_length(first_token, b) >= r1) break;
        const int64_t len = kvstarts[b + 1] - kv_base - first_token;
        const int64_t s_beg = sequence_origin(first_token, b);
        int64_t pa, pe;
        piece_bounds(r0, r1, s_beg, len, kMfmaBlock, pa, pe);
        if (pe <= pa) continue;
        const int pa32 = (int)pa, pe32 = (int)pe;
        const int nb = (pe32 - pa32 + kMfmaBlock - 1) / kMfmaBlock;

        const int64_t table_base = PAGED ? (int64_t)b * a.cachestarts_stride_b : (int64_t)b;
        const int64_t seq_row0 = PAGED ? 0 : cachestarts[b];
        // a block of 32 tokens starts on a multiple of 32 and so lies inside one 128-token page
        auto row_base_of = [&](int pos) -> int64_t {
            if (!PAGED) return seq_row0 + pos;
            return cachestarts[table_base + (pos >> 7)] + (pos & (kPage - 1));
        };

        // ---- Q fragments (B operand of S^T): column = query head l32; k-step s of half-wave hh covers the
        // channels [HALF hh + 16 (s / 2) + 8 (s % 2), + 8), so that a lane's K bytes are HALF consecutive ones ----
        int64_t q_row = b; // row of the query and output tensors
        int qlen = 1;
        if (CHUNK) {
            q_row = a.seqstarts[b];
            qlen = (int)(a.seqstarts[b + 1] - q_row);
        }
        const bool on = gq < G && cpos < qlen;
        // tokens this column attends: all of the sequence, or (causal chunk) those up to its own position
        const int col_lim = CHUNK && a.chunk_causal ? (int)len - qlen + cpos + 1 : (int)len;
        const int first_cut = CHUNK && a.chunk_causal ? (int)len - qlen + 1 : (int)len; // the smallest limit of any column
        f16x8 qf[KS];
        {
            const half_t* qp = (const half_t*)a.query + (q_row + (on ? cpos : 0)) * a.query_stride_s + (int64_t)(kvh * GR + (on ? cg : 0)) * D + HALF * hh;
#pragma unroll
            for (int s = 0; s < KS; ++s) {
                qf[s] = *(const f16x8*)(qp + 8 * s);
                if (!on) {
#pragma unroll
                    for (int e = 0; e < 8; ++e) qf[s][e] = (half_t)0.f;
                }
            }
        }
        const half_t* mask_row = nullptr;
        if (MASK) {
            const int h = kvh * G + (gq < G ? gq : 0);
            mask_row = (const half_t*)a.attn_mask + (int64_t)h * a.mask_stride_h + (int64_t)b * a.mask_stride_s + kvstarts[b];
        }

        // ---- raw bytes of one block: K as (token l32, channels HALF hh .. + HALF), V as (token quad, group) units ----
        u32x4 kq[KW];
        uint32_t ksc[KW]; // two half scales each
        u32x2 vq[VU][4];
        half_t vsc[VU][4];
        // per-lane offsets inside a block: constant except in a piece's last block, whose tokens beyond the
        // piece re-read its last token (their logits are masked)
        uint32_t k_off = (uint32_t)l32 * stride_s32 + HALF * hh;
        uint32_t v_off[VU][4];
#pragma unroll
        for (int u = 0; u < VU; ++u)
#pragma unroll
            for (int r = 0; r < 4; ++r) v_off[u][r] = (uint32_t)(4 * v_q[u] + r) * stride_s32 + 8 * v_g;
        auto clamp_offsets = [&](int pos) {
            const int last = pe32 - 1 - pos; // offset of the piece's last token inside this block (>= 0)
            k_off = (uint32_t)(l32 < last ? l32 : last) * stride_s32 + HALF * hh;
#pragma unroll
            for (int u = 0; u < VU; ++u)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int t = 4 * v_q[u] + r;
                    v_off[u][r] = (uint32_t)(t < last ? t : last) * stride_s32 + 8 * v_g;
                }
        };
        auto load_k = [&](int pos) {
            const int64_t boff = row_base_of(pos) * a.cache_stride_s;
            const char* bk = cache_k + boff;
            const half_t* sk = scale_k + (boff >> 3);
#pragma unroll
            for (int j = 0; j < KW; ++j) {
                kq[j] = *(const u32x4*)(bk + k_off + 16 * j);
                ksc[j] = *(const uint32_t*)(sk + (k_off >> 3) + 2 * j);
            }
        };
        auto load_v = [&](int pos) {
            const int64_t boff = row_base_of(pos) * a.cache_stride_s;
            const char* bv = cache_v + boff;
            const half_t* sv = scale_v + (boff >> 3);
#pragma unroll
            for (int u = 0; u < VU; ++u)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    vq[u][r] = *(const u32x2*)(bv + v_off[u][r]);
                    vsc[u][r] = sv[v_off[u][r] >> 3];
                }
        };

        f32x16 o_acc[CB];
#pragma unroll
        for (int cb = 0; cb < CB; ++cb)
#pragma unroll
            for (int i = 0; i < 16; ++i) o_acc[cb][i] = 0.f;
        float m_run = kNegBig, l_run = 0.f;

        if (pa32 + kMfmaBlock > pe32) clamp_offsets(pa32);
        load_v(pa32);
        load_k(pa32);
        for (int i = 0; i < nb; ++i) {
            const int pos = pa32 + i * kMfmaBlock;

            // ---- V: dequantise (hi + lo halves) and store transposed into the wave's LDS tile ----
            wave_lds_handoff(); // every lane is past its reads of the previous block's tile
#pragma unroll
            for (int u = 0; u < VU; ++u) {
                const half2_t s01 = {vsc[u][0], vsc[u][1]}, s23 = {vsc[u][2], vsc[u][3]};
                const int posv = 16 * (v_q[u] >> 2) + vt_pos16(4 * (v_q[u] & 3));
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    constexpr uint32_t kSel[4] = {0x0c040c00u, 0x0c050c01u, 0x0c060c02u, 0x0c070c03u}; // byte e & 3 of two words
                    const uint32_t sel = kSel[e & 3];
                    const uint32_t w0 = vq[u][0][e >> 2], w1 = vq[u][1][e >> 2], w2 = vq[u][2][e >> 2], w3 = vq[u][3][e >> 2];
                    const half2_t x01 = pk_sub_1152(__builtin_amdgcn_perm(w1, w0, sel) ^ 0x64806480u);
                    const half2_t x23 = pk_sub_1152(__builtin_amdgcn_perm(w3, w2, sel) ^ 0x64806480u);
                    const half2_t h01 = x01 * s01, h23 = x23 * s23;
                    u32x2 out, outl;
                    out[0] = bitcast<uint32_t>(h01);
                    out[1] = bitcast<uint32_t>(h23);
                    outl[0] = bitcast<uint32_t>(__builtin_elementwise_fma(x01, s01, -h01));
                    outl[1] = bitcast<uint32_t>(__builtin_elementwise_fma(x23, s23, -h23));
                    const int idx = vt_index(vt_row(8 * v_g + e), posv);
                    *(u32x2*)&sV[idx] = out;
                    *(u32x2*)&sVlo[idx] = outl;
                }
            }

            wave_lds_handoff(); // the tile is complete before any lane reads it
            // the raw registers are free again: the next block's bytes travel while this one is finished
            if (i + 1 < nb) {
                if (pos + 2 * kMfmaBlock > pe32) clamp_offsets(pos + kMfmaBlock); // the next block is the last and partial
                load_v(pos + kMfmaBlock);
            }

            // ---- S^T = K Q^T: the A fragments are built from this lane's raw bytes step by step ----
            f32x16 s_acc;
#pragma unroll
            for (int e = 0; e < 16; ++e) s_acc[e] = 0.f;
#pragma unroll
            for (int s = 0; s < KS; ++s) {
                const int j = s >> 1, e = s & 1;
                const half_t sc1 = bitcast<half2_t>(ksc[j])[e];
                const half2_t sc = {sc1, sc1};
                const uint32_t f0 = kq[j][2 * e] ^ kFlipSigns, f1 = kq[j][2 * e + 1] ^ kFlipSigns;
                const half2_t x0 = cvt_bytes01(f0), x1 = cvt_bytes23(f0), x2 = cvt_bytes01(f1), x3 = cvt_bytes23(f1);
                const half2_t h0 = x0 * sc, h1 = x1 * sc, h2 = x2 * sc, h3 = x3 * sc;
                const half2_t g0 = __builtin_elementwise_fma(x0, sc, -h0), g1 = __builtin_elementwise_fma(x1, sc, -h1);
                const half2_t g2 = __builtin_elementwise_fma(x2, sc, -h2), g3 = __builtin_elementwise_fma(x3, sc, -h3);
                const f16x8 ah = {h0[0], h0[1], h1[0], h1[1], h2[0], h2[1], h3[0], h3[1]};
                const f16x8 al = {g0[0], g0[1], g1[0], g1[1], g2[0], g2[1], g3[0], g3[1]};
                s_acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(al, qf[s], s_acc, 0, 0, 0);
                s_acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah, qf[s], s_acc, 0, 0, 0);
            }

            if (i + 1 < nb) load_k(pos + kMfmaBlock);

            // ---- online softmax per column (element e <-> token 8 (e / 4) + 4 hh + e % 4) ----
            if (MASK) {
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const int t = pos + 8 * (e >> 2) + 4 * hh + (e & 3);
                    s_acc[e] += (float)mask_row[t < pe32 ? t : pe32 - 1] * (kLog2e / sm_scale);
                }
            }
            if (pos + kMfmaBlock > pe32 || (CHUNK && pos + kMfmaBlock > first_cut)) { // a piece's last block, or one that reaches a column's causal limit (wave-uniform)
                const int lim = CHUNK ? (col_lim < pe32 ? col_lim : pe32) : pe32;
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const int t = pos + 8 * (e >> 2) + 4 * hh + (e & 3);
                    if (t >= lim) s_acc[e] = -INFINITY;
                }
            }
            // maximum of the raw dot products; the (positive) logit scale is applied to it afterwards
            float mx = kNegBig;
#pragma unroll
            for (int e = 0; e < 16; ++e) mx = fmaxf(mx, s_acc[e]);
            mx *= sm_scale;
            mx = fmaxf(mx, __shfl_xor(mx, 32));
            const float m_new = fmaxf(m_run, mx);
            if (__builtin_amdgcn_ballot_w64(m_new > m_run) != 0) { // wave-uniform and rare once a few blocks were seen
                const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
                l_run *= alpha;
#pragma unroll
                for (int cb = 0; cb < CB; ++cb)
#pragma unroll
                    for (int e = 0; e < 16; ++e) o_acc[cb][e] *= alpha;
                m_run = m_new;
            }
            const float bias = kPShift - m_run;
            f16x8 pf[2], pfl[2];
            float lsum = 0.f;
#pragma unroll
            for (int e = 0; e < 16; e += 2) {
                const float p0 = __builtin_amdgcn_exp2f(__builtin_fmaf(s_acc[e], sm_scale, bias));
                const float p1 = __builtin_amdgcn_exp2f(__builtin_fmaf(s_acc[e + 1], sm_scale, bias));
                lsum += p0 + p1;
                const half2_t ph = bitcast<half2_t>(__builtin_amdgcn_cvt_pkrtz(p0, p1));
                const half2_t pl = bitcast<half2_t>(__builtin_amdgcn_cvt_pkrtz(sub_half_lo(p0, ph), sub_half_hi(p1, ph)));
                pf[e >> 3][e & 7] = ph.x;
                pf[e >> 3][(e & 7) + 1] = ph.y;
                pfl[e >> 3][e & 7] = pl.x;
                pfl[e >> 3][(e & 7) + 1] = pl.y;
            }
            l_run += lsum;

            // ---- O^T += V^T P^T ----
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int cb = 0; cb < CB; ++cb) {
                    const int idx = vt_index(vt_row(32 * cb + l32), 16 * t + 8 * hh);
                    const f16x8 vh = *(const f16x8*)&sV[idx];
                    const f16x8 vl = *(const f16x8*)&sVlo[idx];
                    o_acc[cb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vl, pf[t], o_acc[cb], 0, 0, 0);
                    o_acc[cb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vh, pfl[t], o_acc[cb], 0, 0, 0);
                    o_acc[cb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vh, pf[t], o_acc[cb], 0, 0, 0);
                }
        }

        // ---- end of the piece: element e of block cb <-> channel 32 cb + 8 (e / 4) + 4 hh + e % 4 ----
        const float l_tot = l_run + __shfl_xor(l_run, 32);
        const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
        if (on) {
            const int h = kvh * G + gq; // the column among all columns: its slot in the pieces' workspace
            const bool whole = (pa == 0) && (pe == len);
            if (whole) {
                half_t* op = (half_t*)a.output + (q_row + cpos) * a.output_stride_s + (int64_t)(kvh * GR + cg) * D;
#pragma unroll
                for (int cb = 0; cb < CB; ++cb)
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        f16x4 w;
#pragma unroll
                        for (int e = 0; e < 4; ++e) w[e] = (half_t)(o_acc[cb][4 * r + e] * inv);
                        *(f16x4*)(op + 32 * cb + 8 * r + 4 * hh) = w;
                    }
            } else {
                const int64_t piece = (int64_t)blockIdx.x + b;
                float* op = a.partial_out + (piece * a.num_heads + h) * D;
#pragma unroll
                for (int cb = 0; cb < CB; ++cb)
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                        *(f32x4*)(op + 32 * cb + 8 * r + 4 * hh) =
                            f32x4{o_acc[cb][4 * r] * inv, o_acc[cb][4 * r + 1] * inv, o_acc[cb][4 * r + 2] * inv, o_acc[cb][4 * r + 3] * inv};
                if (hh == 0) {
                    a.partial_ml[(piece * a.num_heads + h) * 2 + 0] = m_run;
                    a.partial_ml[(piece * a.num_heads + h) * 2 + 1] = l_tot * 0x1p-14f; // p carries the factor 2^kPShift
                }
            }
        }
    }
}

// The same path for up to sixteen query heads per kv head, on v_mfma_f32_16x16x32_f16: half the columns,
// so half the MFMA time, half the logits per lane and half the accumulator registers.
//   lane = (r = lane % 16, qq = lane / 16)
//   S^T tile (16 tokens x 16 columns, two per block): A = K rows of token 16 tile + r, B = Q of head r;
//     k-step s = 2 j + e pairs the lane's channels [64 j + 16 qq + 8 e, + 8) on both sides
//     (those 16-byte pieces reach the lane through LDS: with this layout a load instruction would read 64 of a
//     row's 128 bytes, so the rows are loaded as whole lines by eight lanes each, with the non-temporal hint,
//     and the block's 4 KB pass through a wave-private LDS buffer);
//     the accumulator holds tokens 16 tile + 4 qq + i of column r
//   O^T tile (16 channels x 16 columns, eight per block): A = row `channel 16 cb + r` of the V^T tile,
//     16-byte block qq, whose eight positions are the tokens of the lane's two S^T accumulators in order:
//     position 8 qq + 4 tile + i <-> token 16 tile + 4 qq + i; the accumulator holds channels 16 cb + 4 qq + i
// CHUNK: as in the 32-column kernel (columns = (query position, query head) pairs of short chunks).
template <int NW, bool PAGED, bool MASK, bool CHUNK = false>
__global__ __launch_bounds__(NW * kWave, 2) void decode_attention_mfma16_kernel(const DecodeLaunch a)
{
    static_assert(!(CHUNK && MASK), "no attn_mask form for chunks");
    constexpr int D = kMfmaD;
    __shared__ __attribute__((aligned(16))) half_t s_vt[NW][2][D * kMfmaBlock]; // [wave][hi, lo]
    // a block's raw K rows, on their way from whole-line loads to the lanes that hold them as MFMA operands:
    // row = token, eight 16-byte chunks per row, chunk index XORed with (token ^ token >> 3) & 7 (no bank conflicts)
    __shared__ __attribute__((aligned(16))) char s_k[NW][kMfmaBlock * D];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r16 = lane & 15;
    const int qq = lane >> 4;
    const int G = (int)a.num_kv_repeats;
    const int GR = CHUNK ? (int)a.chunk_q_heads : G;       // query heads per kv head
    const int cpos = CHUNK ? r16 / GR : 0;                 // the column's query position within its sequence's chunk
    const int cg = CHUNK ? r16 - cpos * GR : r16;          // ... and its query head within the kv head's group
    const int kvh = blockIdx.y * NW + wave;
    half_t* const sV = s_vt[wave][0];
    half_t* const sVlo = s_vt[wave][1];
    char* const sK = s_k[wave];

    const const_i64_ptr kvstarts = as_constant(a.kvstarts);
    const const_i64_ptr cachestarts = as_constant(a.cachestarts);
    const int64_t kv_base = kvstarts[0];
    const int64_t total = stream_length(kvstarts[a.decoding_batches] - kv_base, a.decoding_batches);
    const int64_t per = tokens_per_range(total, a.ranges, kMfmaBlock, a.min_tokens_per_range);
    const int64_t r0 = (int64_t)blockIdx.x * per;
    if (r0 >= total) return;
    const int64_t r1 = (r0 + per < total) ? r0 + per : total;

    const int64_t head_off = a.layer_idx * a.cache_stride_l + (int64_t)kvh * a.cache_stride_h;
    const uint32_t stride_s32 = (uint32_t)a.cache_stride_s; // the host checks that a block's span fits 32 bits
    const char* const cache_k = (const char*)a.cache + head_off;
    const char* const cache_v = cache_k + a.cache_stride_kv;
    const half_t* const scale_k = (const half_t*)a.scale + (head_off >> 3);
    const half_t* const scale_v = scale_k + (a.cache_stride_kv >> 3);
    const float sm_scale = a.attn_scale * kLog2e;

    // V units of this lane: the eight channels of group v_g for two token quads (tokens 4 q .. + 4, which the
    // V^T tile holds at positions 8 (q % 4) + 4 (q / 4) .. + 4).  The lanes of one store instruction alternate
    // between the two 8-byte halves of the 16-byte blocks, so that they cover all banks.
    const int v_g = lane & 15;
    int v_q[2];
    v_q[0] = qq + 4 * (qq & 1);
    v_q[1] = qq + 4 * ((qq & 1) ^ 1);

    int b = find_sequence(kvstarts, a.kvstarts, (int)a.decoding_batches, r0, lane);
    for (; b < a.decoding_batches; ++b) {
        const int64_t first_token = kvstarts[b] - kv_base;
        if (stream_length(first_token, b) >= r1) break;
        const int64_t len = kvstarts[b + 1] - kv_base - first_token;
        const int64_t s_beg = sequence_origin(first_token, b);
        int64_t pa, pe;
        piece_bounds(r0, r1, s_beg, len, kMfmaBlock, pa, pe);
        if (pe <= pa) continue;
        const int pa32 = (int)pa, pe32 = (int)pe;
        const int nb = (pe32 - pa32 + kMfmaBlock - 1) / kMfmaBlock;

        const int64_t table_base = PAGED ? (int64_t)b * a.cachestarts_stride_b : (int64_t)b;
        const int64_t seq_row0 = PAGED ? 0 : cachestarts[b];
        // a block of 32 tokens starts on a multiple of 32 and so lies inside one 128-token page
        auto row_base_of = [&](int pos) -> int64_t {
            if (!PAGED) return seq_row0 + pos;
            return cachestarts[table_base + (pos >> 7)] + (pos & (kPage - 1));
        };

        // ---- Q fragments (B operand of S^T): column = query head r16 ----
        int64_t q_row = b; // row of the query and output tensors
        int qlen = 1;
        if (CHUNK) {
            q_row = a.seqstarts[b];
            qlen = (int)(a.seqstarts[b + 1] - q_row);
        }
        const bool on = r16 < G && cpos < qlen;
        // tokens this column attends: all of the sequence, or (causal chunk) those up to its own position
        const int col_lim = CHUNK && a.chunk_causal ? (int)len - qlen + cpos + 1 : (int)len;
        const int first_cut = CHUNK && a.chunk_causal ? (int)len - qlen + 1 : (int)len; // the smallest limit of any column
        f16x8 qf[4];
        {
            const half_t* qp = (const half_t*)a.query + (q_row + (on ? cpos : 0)) * a.query_stride_s + (int64_t)(kvh * GR + (on ? cg : 0)) * D + 16 * qq;
#pragma unroll
            for (int s = 0; s < 4; ++s) {
                qf[s] = *(const f16x8*)(qp + 64 * (s >> 1) + 8 * (s & 1));
                if (!on) {
#pragma unroll
                    for (int e = 0; e < 8; ++e) qf[s][e] = (half_t)0.f;
                }
            }
        }
        const half_t* mask_row = nullptr;
        if (MASK) {
            const int h = kvh * G + (r16 < G ? r16 : 0);
            mask_row = (const half_t*)a.attn_mask + (int64_t)h * a.mask_stride_h + (int64_t)b * a.mask_stride_s + kvstarts[b];
        }

        // ---- raw bytes of one block: K of tokens r16 and 16 + r16, V as two (token quad, group) units ----
        u32x4 kq[2][2];
        u32x4 kraw[4];      // K as loaded: token 8 i + lane / 8, channels 16 (lane % 8) .. + 16 (whole lines per instruction)
        uint32_t ksc[2][2]; // two half scales each
        u32x2 vq[2][4];
        half_t vsc[2][4];
        // per-lane offsets inside a block: constant except in a piece's last block, whose tokens beyond the
        // piece re-read its last token (their logits are masked)
        uint32_t k_off[2];
        uint32_t kl_off[4];
        uint32_t v_off[2][4];
#pragma unroll
        for (int t = 0; t < 2; ++t) k_off[t] = (uint32_t)(16 * t + r16) * stride_s32 + 16 * qq;
#pragma unroll
        for (int i4 = 0; i4 < 4; ++i4) kl_off[i4] = (uint32_t)(8 * i4 + (lane >> 3)) * stride_s32 + 16 * (lane & 7);
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
            for (int r = 0; r < 4; ++r) v_off[u][r] = (uint32_t)(4 * v_q[u] + r) * stride_s32 + 8 * v_g;
        auto clamp_offsets = [&](int pos) {
            const int last = pe32 - 1 - pos; // offset of the piece's last token inside this block (>= 0)
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                const int tk = 16 * t + r16;
                k_off[t] = (uint32_t)(tk < last ? tk : last) * stride_s32 + 16 * qq;
            }
#pragma unroll
            for (int i4 = 0; i4 < 4; ++i4) {
                const int tk = 8 * i4 + (lane >> 3);
                kl_off[i4] = (uint32_t)(tk < last ? tk : last) * stride_s32 + 16 * (lane & 7);
            }
#pragma unroll
            for (int u = 0; u < 2; ++u)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int t = 4 * v_q[u] + r;
                    v_off[u][r] = (uint32_t)(t < last ? t : last) * stride_s32 + 8 * v_g;
                }
        };
        auto load_k = [&](int pos) {
            const int64_t boff = row_base_of(pos) * a.cache_stride_s;
            const char* bk = cache_k + boff;
            const half_t* sk = scale_k + (boff >> 3);
#pragma unroll
            for (int i4 = 0; i4 < 4; ++i4) kraw[i4] = __builtin_nontemporal_load((const u32x4*)(bk + kl_off[i4]));
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int j = 0; j < 2; ++j) ksc[t][j] = *(const uint32_t*)(sk + (k_off[t] >> 3) + 8 * j);
        };
        // through the wave's LDS rows to the operand layout: lane (r16, qq) takes channels 64 j + 16 qq .. + 16 of the
        // tokens r16 and 16 + r16 (the wave's LDS operations execute in order: no workgroup barrier, only the
        // compiler is told about the hand-off)
        auto stage_k = [&]() {
            wave_lds_handoff(); // every lane is past its reads of the previous block's rows
#pragma unroll
            for (int i4 = 0; i4 < 4; ++i4) {
                const int tk = 8 * i4 + (lane >> 3);
                *(u32x4*)(sK + tk * D + ((((lane & 7) ^ tk ^ (tk >> 3)) & 7) << 4)) = kraw[i4];
            }
            wave_lds_handoff(); // rows stored by eight lanes each, read back by the lanes that hold them as operands
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    const int tk = 16 * t + r16;
                    kq[t][j] = *(const u32x4*)(sK + tk * D + ((((4 * j + qq) ^ tk ^ (tk >> 3)) & 7) << 4));
                }
        };
        auto load_v = [&](int pos) {
            const int64_t boff = row_base_of(pos) * a.cache_stride_s;
            const char* bv = cache_v + boff;
            const half_t* sv = scale_v + (boff >> 3);
#pragma unroll
            for (int u = 0; u < 2; ++u)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    vq[u][r] = __builtin_nontemporal_load((const u32x2*)(bv + v_off[u][r]));
                    vsc[u][r] = sv[v_off[u][r] >> 3];
                }
        };
        // only a piece's last block can be partial, and it is the last one loaded
        f32x4 o_acc[8];
#pragma unroll
        for (int cb = 0; cb < 8; ++cb)
#pragma unroll
            for (int i = 0; i < 4; ++i) o_acc[cb][i] = 0.f;
        float m_run = kNegBig, l_run = 0.f;

        if (pa32 + kMfmaBlock > pe32) clamp_offsets(pa32);
        load_v(pa32);
        load_k(pa32);
        for (int i = 0; i < nb; ++i) {
            const int pos = pa32 + i * kMfmaBlock;

            // ---- V: dequantise (hi + lo halves) and store transposed into the wave's LDS tile ----
            // (8-byte stores of the two tiles pair up into one instruction; 16-byte stores of a channel's eight
            // tokens take the same time)
            wave_lds_handoff(); // every lane is past its reads of the previous block's tile
#pragma unroll
            for (int u = 0; u < 2; ++u) {
                const half2_t s01 = {vsc[u][0], vsc[u][1]}, s23 = {vsc[u][2], vsc[u][3]};
                const int posv = 8 * (v_q[u] & 3) + 4 * (v_q[u] >> 2);
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    constexpr uint32_t kSel[4] = {0x0c040c00u, 0x0c050c01u, 0x0c060c02u, 0x0c070c03u}; // byte e & 3 of two words
                    const uint32_t sel = kSel[e & 3];
                    const uint32_t w0 = vq[u][0][e >> 2], w1 = vq[u][1][e >> 2], w2 = vq[u][2][e >> 2], w3 = vq[u][3][e >> 2];
                    const half2_t x01 = pk_sub_1152(__builtin_amdgcn_perm(w1, w0, sel) ^ 0x64806480u);
                    const half2_t x23 = pk_sub_1152(__builtin_amdgcn_perm(w3, w2, sel) ^ 0x64806480u);
                    const half2_t h01 = x01 * s01, h23 = x23 * s23;
                    u32x2 out, outl;
                    out[0] = bitcast<uint32_t>(h01);
                    out[1] = bitcast<uint32_t>(h23);
                    outl[0] = bitcast<uint32_t>(__builtin_elementwise_fma(x01, s01, -h01));
                    outl[1] = bitcast<uint32_t>(__builtin_elementwise_fma(x23, s23, -h23));
                    const int idx = vt_index(vt_row(8 * v_g + e), posv);
                    *(u32x2*)&sV[idx] = out;
                    *(u32x2*)&sVlo[idx] = outl;
                }
            }

            wave_lds_handoff(); // the tile is complete before any lane reads it
            // the raw registers are free again: the next block's bytes travel while this one is finished
            if (i + 1 < nb) {
                if (pos + 2 * kMfmaBlock > pe32) clamp_offsets(pos + kMfmaBlock); // the next block is the last and partial
                load_v(pos + kMfmaBlock);
            }

            // ---- S^T = K Q^T: the A fragments are built from this lane's raw bytes step by step ----
            stage_k();
            f32x4 s_acc[2];
#pragma unroll
            for (int t = 0; t < 2; ++t) {
#pragma unroll
                for (int e = 0; e < 4; ++e) s_acc[t][e] = 0.f;
#pragma unroll
                for (int s = 0; s < 4; ++s) {
                    const int j = s >> 1, e = s & 1;
                    const half_t sc1 = bitcast<half2_t>(ksc[t][j])[e];
                    const half2_t sc = {sc1, sc1};
                    const uint32_t f0 = kq[t][j][2 * e] ^ kFlipSigns, f1 = kq[t][j][2 * e + 1] ^ kFlipSigns;
                    const half2_t x0 = cvt_bytes01(f0), x1 = cvt_bytes23(f0), x2 = cvt_bytes01(f1), x3 = cvt_bytes23(f1);
                    const half2_t h0 = x0 * sc, h1 = x1 * sc, h2 = x2 * sc, h3 = x3 * sc;
                    const half2_t g0 = __builtin_elementwise_fma(x0, sc, -h0), g1 = __builtin_elementwise_fma(x1, sc, -h1);
                    const half2_t g2 = __builtin_elementwise_fma(x2, sc, -h2), g3 = __builtin_elementwise_fma(x3, sc, -h3);
                    const f16x8 ah = {h0[0], h0[1], h1[0], h1[1], h2[0], h2[1], h3[0], h3[1]};
                    const f16x8 al = {g0[0], g0[1], g1[0], g1[1], g2[0], g2[1], g3[0], g3[1]};
                    s_acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(al, qf[s], s_acc[t], 0, 0, 0);
                    s_acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ah, qf[s], s_acc[t], 0, 0, 0);
                }
            }

            if (i + 1 < nb) load_k(pos + kMfmaBlock);

            // ---- online softmax per column (element e of tile t <-> token 16 t + 4 qq + e) ----
            if (MASK) {
#pragma unroll
                for (int t = 0; t < 2; ++t)
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const int tk = pos + 16 * t + 4 * qq + e;
                        s_acc[t][e] += (float)mask_row[tk < pe32 ? tk : pe32 - 1] * (kLog2e / sm_scale);
                    }
            }
            if (pos + kMfmaBlock > pe32 || (CHUNK && pos + kMfmaBlock > first_cut)) { // a piece's last block, or one that reaches a column's causal limit (wave-uniform)
                const int lim = CHUNK ? (col_lim < pe32 ? col_lim : pe32) : pe32;
#pragma unroll
                for (int t = 0; t < 2; ++t)
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const int tk = pos + 16 * t + 4 * qq + e;
                        if (tk >= lim) s_acc[t][e] = -INFINITY;
                    }
            }
            // maximum of the raw dot products; the (positive) logit scale is applied to it afterwards
            float mx = kNegBig;
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int e = 0; e < 4; ++e) mx = fmaxf(mx, s_acc[t][e]);
            mx *= sm_scale;
            mx = fmaxf(mx, __shfl_xor(mx, 16));
            mx = fmaxf(mx, __shfl_xor(mx, 32));
            const float m_new = fmaxf(m_run, mx);
            if (__builtin_amdgcn_ballot_w64(m_new > m_run) != 0) { // wave-uniform and rare once a few blocks were seen
                const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
                l_run *= alpha;
#pragma unroll
                for (int cb = 0; cb < 8; ++cb)
#pragma unroll
                    for (int e = 0; e < 4; ++e) o_acc[cb][e] *= alpha;
                m_run = m_new;
            }
            const float bias = kPShift - m_run;
            f16x8 pf, pfl;
            float lsum = 0.f;
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int e = 0; e < 4; e += 2) {
                    const float p0 = __builtin_amdgcn_exp2f(__builtin_fmaf(s_acc[t][e], sm_scale, bias));
                    const float p1 = __builtin_amdgcn_exp2f(__builtin_fmaf(s_acc[t][e + 1], sm_scale, bias));
                    lsum += p0 + p1;
                    const half2_t ph = bitcast<half2_t>(__builtin_amdgcn_cvt_pkrtz(p0, p1));
                    const half2_t pl = bitcast<half2_t>(__builtin_amdgcn_cvt_pkrtz(sub_half_lo(p0, ph), sub_half_hi(p1, ph)));
                    pf[4 * t + e] = ph.x;
                    pf[4 * t + e + 1] = ph.y;
                    pfl[4 * t + e] = pl.x;
                    pfl[4 * t + e + 1] = pl.y;
                }
            l_run += lsum;

            // ---- O^T += V^T P^T ----
#pragma unroll
            for (int cb = 0; cb < 8; ++cb) {
                const int idx = vt_index(vt_row(16 * cb + r16), 8 * qq);
                const f16x8 vh = *(const f16x8*)&sV[idx];
                const f16x8 vl = *(const f16x8*)&sVlo[idx];
                o_acc[cb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(vl, pf, o_acc[cb], 0, 0, 0);
                o_acc[cb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(vh, pfl, o_acc[cb], 0, 0, 0);
                o_acc[cb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(vh, pf, o_acc[cb], 0, 0, 0);
            }
        }

        // ---- end of the piece: element e of tile cb <-> channel 16 cb + 4 qq + e ----
        float l_tot = l_run + __shfl_xor(l_run, 16);
        l_tot += __shfl_xor(l_tot, 32);
        const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
        if (on) {
            const int h = kvh * G + r16; // the column among all columns: its slot in the pieces' workspace
            const bool whole = (pa == 0) && (pe == len);
            if (whole) {
                half_t* op = (half_t*)a.output + (q_row + cpos) * a.output_stride_s + (int64_t)(kvh * GR + cg) * D;
#pragma unroll
                for (int cb = 0; cb < 8; ++cb) {
                    f16x4 w;
#pragma unroll
                    for (int e = 0; e < 4; ++e) w[e] = (half_t)(o_acc[cb][e] * inv);
                    *(f16x4*)(op + 16 * cb + 4 * qq) = w;
                }
            } else {
                const int64_t piece = (int64_t)blockIdx.x + b;
                float* op = a.partial_out + (piece * a.num_heads + h) * D;
#pragma unroll
                for (int cb = 0; cb < 8; ++cb)
                    *(f32x4*)(op + 16 * cb + 4 * qq) =
                        f32x4{o_acc[cb][0] * inv, o_acc[cb][1] * inv, o_acc[cb][2] * inv, o_acc[cb][3] * inv};
                if (qq == 0) {
                    a.partial_ml[(piece * a.num_heads + h) * 2 + 0] = m_run;
                    a.partial_ml[(piece * a.num_heads + h) * 2 + 1] = l_tot * 0x1p-14f; // p carries the factor 2^kPShift
                }
            }
        }
    }
}

template <int NW, int D>
static void launch_decode_mfma32(const DecodeLaunch& a, dim3 grid, dim3 block, hipStream_t stream)
{
    const bool paged = a.cache_mode == 1, mask = a.attn_mask != nullptr;
    if (a.seqstarts != nullptr) { // chunks of query tokens (no mask form: the caller checks)
        if (paged) hipLaunchKernelGGL((decode_attention_mfma_kernel<NW, true, false, D, true>), grid, block, 0, stream, a);
        else hipLaunchKernelGGL((decode_attention_mfma_kernel<NW, false, false, D, true>), grid, block, 0, stream, a);
        return;
    }
    if (paged) {
        if (mask) hipLaunchKernelGGL((decode_attention_mfma_kernel<NW, true, true, D>), grid, block, 0, stream, a);
        else hipLaunchKernelGGL((decode_attention_mfma_kernel<NW, true, false, D>), grid, block, 0, stream, a);
    } else {
        if (mask) hipLaunchKernelGGL((decode_attention_mfma_kernel<NW, false, true, D>), grid, block, 0, stream, a);
        else hipLaunchKernelGGL((decode_attention_mfma_kernel<NW, false, false, D>), grid, block, 0, stream, a);
    }
}

template <int NW>
static void launch_decode_mfma_nw(const DecodeLaunch& a, hipStream_t stream)
{
    const dim3 grid((unsigned)a.ranges, (unsigned)(a.num_kv_heads / NW), 1);
    const dim3 block(NW * kWave);
    const bool paged = a.cache_mode == 1, mask = a.attn_mask != nullptr;
    if (a.kernel == kDecodeKernelMfma16) {
        if (a.seqstarts != nullptr) { // chunks of query tokens (no mask form: the caller checks)
            if (paged) hipLaunchKernelGGL((decode_attention_mfma16_kernel<NW, true, false, true>), grid, block, 0, stream, a);
            else hipLaunchKernelGGL((decode_attention_mfma16_kernel<NW, false, false, true>), grid, block, 0, stream, a);
            return;
        }
        if (paged) {
            if (mask) hipLaunchKernelGGL((decode_attention_mfma16_kernel<NW, true, true>), grid, block, 0, stream, a);
            else hipLaunchKernelGGL((decode_attention_mfma16_kernel<NW, true, false>), grid, block, 0, stream, a);
        } else {
            if (mask) hipLaunchKernelGGL((decode_attention_mfma16_kernel<NW, false, true>), grid, block, 0, stream, a);
            else hipLaunchKernelGGL((decode_attention_mfma16_kernel<NW, false, false>), grid, block, 0, stream, a);
        }
        return;
    }
    // the 32-column form: head_dim 128 or 64, and as many passes as the query heads of a kv head need
    const dim3 grid32((unsigned)a.ranges, (unsigned)(a.num_kv_heads / NW), (unsigned)a.num_passes);
    if (a.head_dim == 64) launch_decode_mfma32<NW, 64>(a, grid32, block, stream);
    else launch_decode_mfma32<NW, 128>(a, grid32, block, stream);
}

void launch_decode_mfma(const DecodeLaunch& a, hipStream_t stream)
{
    switch (a.kv_heads_per_group) { // a wave per kv head
    case 4: launch_decode_mfma_nw<4>(a, stream); break;
    case 2: launch_decode_mfma_nw<2>(a, stream); break;
    default: launch_decode_mfma_nw<1>(a, stream); break;
    }
}

} // namespace pmxhip
