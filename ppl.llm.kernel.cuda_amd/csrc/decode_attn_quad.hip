// Decode attention over the int8 group-8 KV cache, variant for head_dim 64 and 128 (two or more kv heads; with an
// odd number the last half-wave idles) and 256, up to four query heads per kv head (MHA and the common GQA shapes;
// up to eight at head_dim 256, and at head_dim 128 with kv heads in eights).  Same semantics, token ranges, pieces and workspace as decode_attn.hip
// (reference: src/ppl/kernel/llm/cuda/pmx/multi_head_cache_attention/kernel.cu:229-679,
// 1115-1891); what differs is the lane layout, chosen so that the matrix pipe computes
// the q.k products while the vector pipe converts and accumulates:
//
//   * A wave owns two kv heads and up to four of their query heads; with more than four query
//     heads per kv head a second set of four waves takes heads 4..7 of the same kv heads; a
//     barrier per pair of blocks keeps the two sets within a block of each other, so that the
//     second request for a cache line is served by the cache levels (without it the sets drift
//     apart and HBM is read twice).  The four lanes of a quad hold four different TOKENS of the
//     same 16 channels; the eight quads of a half-wave hold the eight 16-channel chunks of
//     those tokens; the two half-waves hold the two kv heads.  A block is 16 tokens: step j
//     of a lane is token 4 j + (lane in quad).
//   * v_mfma_f32_4x4x4_16b_f16 multiplies, per quad, a 4 x 4 A (row i from lane i) by a 4 x 4
//     B (column j from lane j).  Row i = query head i (its 4 channels), column j = token j
//     (the same 4 channels of K, converted int8 -> 1152 + x halves): one instruction gives
//     each lane the four heads' partial dot products of its own token.  Two instructions
//     cover one 8-channel scale group; the accumulator starts at -1152 * sum(q), which
//     removes the conversion bias.
//   * The partial logits (4 heads x 4 steps per lane, over 16 channels) are summed over the
//     eight chunk lanes by a reduce-scatter (DPP adds with bank masks, a row swap), which
//     leaves two complete logits per lane; exp2 runs on those; an all-gather hands every
//     lane the 16 probabilities of its own tokens.  Lanes keep the heads in a lane-local
//     order (slot s = head (own head) ^ s), so the gather needs no selects.
//   * PV is per lane: int8 -> fp32 exactly, weights p * scale in fp32, v_fmac_f32.  Each lane
//     accumulates its own token stream; the four streams of a quad are merged at the end of
//     a piece.  Waves never exchange data: no LDS, no barriers.
#include "decode_common.h"

namespace pmxhip {

namespace {

typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));

constexpr int kQuadBlock = 16;  // tokens per block
constexpr int kDppRor8 = 0x128; // row_ror:8 = lane ^ 8 inside a row of 16

// exchanges the odd rows (of 16 lanes) of x with the even rows of y
__device__ __forceinline__ void swap_rows(float& x, float& y)
{
    const u32x2_t r = __builtin_amdgcn_permlane16_swap(bitcast<uint32_t>(x), bitcast<uint32_t>(y), false, false);
    x = bitcast<float>(r[0]);
    y = bitcast<float>(r[1]);
}
// value of lane ^ 4 (data-share crossbar, no LDS memory involved): and 0x1f, or 0, xor 4
__device__ __forceinline__ float lane_xor4(float v)
{
    return bitcast<float>(__builtin_amdgcn_ds_swizzle(bitcast<int>(v), (4 << 10) | 0x1f));
}
// lo + lo(lane ^ 4) on lanes with bit 2 clear, hi + hi(lane ^ 4) on lanes with bit 2 set.  The two
// instructions write complementary banks of four lanes.  (A DPP operand must not be read within two
// wait states of its producer; the compiler cannot see into the statement, hence the s_nop.)
__device__ __forceinline__ float fold_xor4(float lo, float hi)
{
    float r;
    asm("s_nop 1\n\t"
        "v_add_f32_dpp %0, %1, %1 row_shl:4 row_mask:0xf bank_mask:0x5\n\t"
        "v_add_f32_dpp %0, %2, %2 row_shr:4 row_mask:0xf bank_mask:0xa"
        : "=&v"(r)
        : "v"(lo), "v"(hi));
    return r;
}
// lo + lo(lane ^ 8) on lanes with bit 3 clear, hi + hi(lane ^ 8) on lanes with bit 3 set
__device__ __forceinline__ float fold_xor8(float lo, float hi)
{
    float r;
    asm("s_nop 1\n\t"
        "v_add_f32_dpp %0, %1, %1 row_ror:8 row_mask:0xf bank_mask:0x3\n\t"
        "v_add_f32_dpp %0, %2, %2 row_ror:8 row_mask:0xf bank_mask:0xc"
        : "=&v"(r)
        : "v"(lo), "v"(hi));
    return r;
}
// v + v(lane ^ 32): the swap hands every lane the value of its own lane in the lower and in the upper half-wave
__device__ __forceinline__ float sum_halves(float v)
{
    const u32x2_t r = __builtin_amdgcn_permlane32_swap(bitcast<uint32_t>(v), bitcast<uint32_t>(v), false, false);
    return bitcast<float>(r[0]) + bitcast<float>(r[1]);
}
// value of the lane with bits 2 and 3 cleared (the chunk lane that holds head 0): and 0x13, or 0, xor 0
__device__ __forceinline__ float from_head0_lane(float v)
{
    return bitcast<float>(__builtin_amdgcn_ds_swizzle(bitcast<int>(v), 0x13));
}
// value held by quad lane i (compile-time i)
template <int I>
__device__ __forceinline__ float quad_lane(float v)
{
    return dpp_f32<I | (I << 2) | (I << 4) | (I << 6)>(v);
}

} // namespace

// GP: sets of four query heads per kv head (1 or 2); WP: pairs of kv heads per workgroup (4, 2 or 1); the workgroup
// has WP * GP waves.  MASK: the additive attn_mask (kernel.cu:319-325), two more requests per block and lane.
// HD: head_dim 128, or 256: the two half-waves then hold the two halves of ONE kv head's channels instead of two kv
// heads, and a logit is the sum of the two half-waves' sums; or 64: a kv head has four chunk lanes, so the two rows of a
// half-wave are two groups of tokens (a block is 32 tokens, step j of a lane is token 16 (row) + 4 j + (lane in quad)),
// the reduce-scatter ends after its two folds with four complete logits per lane, and the rows' token streams are
// merged with the quad's at the end of a piece.
// NS: head slots a lane accumulates: 4, or 1 when every kv head has ONE query head (MHA): the lanes that hold the
// complete logits of the three absent heads then take head 0's probabilities (one swizzle per value instead of the
// all-gather) and a single set of 16 accumulators -- a quarter of the PV arithmetic.
template <bool PAGED, int GP, int WP, bool MASK, int HD, int NS = 4>
__global__ __launch_bounds__(kWave * WP * GP, 2) void decode_attention_quad_kernel(const DecodeLaunch a)
{
    constexpr int D = HD;
    constexpr int KPW = HD == 256 ? 1 : 2; // kv heads per wave
    constexpr bool H64 = HD == 64;         // four channel chunks per kv head: lane bit 4 is a second token group
    constexpr int BLK = H64 ? 2 * kQuadBlock : kQuadBlock; // tokens per block
    static_assert(!(H64 && (MASK || GP > 1)), "head_dim 64: one set of waves, no mask");
    constexpr bool ONE = NS == 1;
    static_assert(NS == 4 || (NS == 1 && GP == 1), "head slots");
    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave_id = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wave = wave_id % WP;      // which pair of kv heads
    const int g_first = (wave_id / WP) * 4; // first query head (within the kv head's group) of this wave
    const int t4 = lane & 3;           // token within a step
    const int chunk = (lane >> 2) & (H64 ? 3 : 7); // channels [16 chunk, 16 chunk + 16)
    const int hsel = lane >> 5;        // which of the wave's two kv heads (head_dim 256: which half of the channels)
    // the head whose complete logits this lane receives from the reduce-scatter
    const int g_own = (((lane >> 2) & 1) << 1) | ((lane >> 3) & 1);
    const int row_odd = (lane >> 4) & 1; // head_dim 64: the token group, tokens 16 row_odd + 4 j + t4 of a block
    const int tok0 = t4 + (H64 ? 16 * row_odd : 0); // this lane's token of step 0
    const int G = (int)a.num_kv_repeats; // <= 4 * GP
    // An odd number of kv heads leaves the last half-wave of the last workgroup without one: it repeats its
    // neighbour's work (the same addresses, so no further memory traffic) and stores nothing.
    const int slot_raw = wave * KPW + (KPW == 2 ? hsel : 0); // kv head within the workgroup
    const bool head_on = blockIdx.y * (KPW * WP) + slot_raw < (int)a.num_kv_heads;
    const int head_slot = head_on ? slot_raw : slot_raw - 1;
    const int kvh = blockIdx.y * (KPW * WP) + head_slot;
    const int ch0 = chunk * 16 + (KPW == 1 ? hsel * 128 : 0); // this lane's 16 channels

    const const_i64_ptr kvstarts = as_constant(a.kvstarts);
    const const_i64_ptr cachestarts = as_constant(a.cachestarts);
    const int64_t kv_base = kvstarts[0];
    const int64_t total = stream_length(kvstarts[a.decoding_batches] - kv_base, a.decoding_batches);
    const int64_t per = tokens_per_range(total, a.ranges, BLK, a.min_tokens_per_range);
    const int64_t r0 = (int64_t)blockIdx.x * per;
    if (r0 >= total) return;
    const int64_t r1 = (r0 + per < total) ? r0 + per : total;

    // Addressing: a 64-bit base per wave (scalar registers) that carries the layer and the wave's first kv head, and
    // a 32-bit offset per lane: (token in block) * stride_s + (second kv head of the wave ? stride_h : 0) + channel.
    // Only one stride_h is left in the lane offset, so a layout that keeps the heads far apart (L, KVH, S, 2, D)
    // is addressed like any other.
    const int64_t group_off = a.layer_idx * a.cache_stride_l + (int64_t)(blockIdx.y * (KPW * WP) + wave * KPW) * a.cache_stride_h;
    const uint32_t stride_s32 = (uint32_t)a.cache_stride_s; // the host checks that a block's span fits 32 bits
    const uint32_t lane_base = (uint32_t)((int64_t)(head_slot - wave * KPW) * a.cache_stride_h + ch0);
    const char* const cache_k = (const char*)a.cache + group_off;
    const char* const cache_v = cache_k + a.cache_stride_kv;
    const char* const scale_k = (const char*)a.scale + (group_off >> 3) * 2;
    const char* const scale_v = scale_k + (a.cache_stride_kv >> 3) * 2;
    const float logit_scale = a.attn_scale * kLog2e;

    // The index entries of a sequence are read one sequence ahead (the first one's come out of the search): a piece
    // that follows another in the range starts at its sequence's first token, so kvstarts and the first page table
    // entry (contiguous cache: the sequence's first row) are known when the piece before it begins, and its first
    // cache rows are requested without a dependent load in front of them.
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
        int64_t pa, pe;
        piece_bounds(r0, r1, s_beg, len, BLK, pa, pe);
        if (pe <= pa) continue;
        const int pa32 = (int)pa, pe32 = (int)pe;
        const int nb = (pe32 - pa32 + BLK - 1) / BLK; // >= 1
        const bool tail_partial = ((pe32 - pa32) & (BLK - 1)) != 0;

        const int64_t table_base = PAGED ? (int64_t)b * a.cachestarts_stride_b : (int64_t)b;
        const int64_t seq_row0 = PAGED ? 0 : (have_first_row ? first_row : cachestarts[b]);
        const int last_page = (pe32 - 1) >> 7;
        // paged: the row of page 0 read ahead stands in as the "next page" of page -1
        int page_idx = have_first_row ? -1 : -2;
        int64_t page_row = 0, next_row = first_row;
        auto row_base_of = [&](int pos) -> int64_t { // page table entries are read one page ahead
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

        uint32_t vo[kTB], vo_sc[kTB];
#pragma unroll
        for (int j = 0; j < kTB; ++j) {
            vo[j] = (uint32_t)(4 * j + tok0) * stride_s32 + lane_base;
            vo_sc[j] = vo[j] >> 2;
        }
        // attn_mask: this lane's two complete logits belong to head g_own and the tokens 4 row_odd + t4 and + 8 of the
        // block; byte offsets against a wave-uniform base (the host checks that they fit 32 bits)
        const char* mask_base = nullptr;
        uint32_t mo[2] = {0, 0};
        uint32_t mask_head = 0;
        if (MASK) {
            const int g = g_first + g_own;
            const int h = kvh * G + (g < G ? g : 0);
            mask_head = (uint32_t)((int64_t)h * a.mask_stride_h * 2);
            mask_base = (const char*)a.attn_mask + ((int64_t)b * a.mask_stride_s + seq_start) * 2;
            mo[0] = mask_head + (uint32_t)(4 * row_odd + t4) * 2;
            mo[1] = mo[0] + 16;
        }
        auto clamp_offsets = [&](int pos) { // tokens beyond the piece re-read its last token; their logits are masked
#pragma unroll
            for (int j = 0; j < kTB; ++j) {
                const int t = pos + 4 * j + tok0;
                const int tc = t < pe32 ? t : pe32 - 1;
                vo[j] = (uint32_t)(tc - pos) * stride_s32 + lane_base;
                vo_sc[j] = vo[j] >> 2;
            }
            if (MASK) {
#pragma unroll
                for (int r = 0; r < 2; ++r) {
                    const int t = pos + 4 * row_odd + t4 + 8 * r;
                    mo[r] = mask_head + (uint32_t)((t < pe32 ? t : pe32 - 1) - pos) * 2;
                }
            }
        };
        // (the row loads carry the non-temporal hint unless a second set of waves reads the same lines)
        auto request_k = [&](KBlock& kb, uint32_t (&mk)[2], int pos) {
            kb.pos = pos;
            const int64_t boff = row_base_of(pos) * a.cache_stride_s;
            kb.boff = boff;
            const char* bk = cache_k + boff;
            const char* sk = scale_k + (boff >> 3) * 2;
#pragma unroll
            for (int j = 0; j < kTB; ++j) {
                load_b128<GP == 1>(kb.q8[j], vo[j], bk);
                load_b32<false>(kb.sc[j], vo_sc[j], sk);
            }
            if (MASK) {
                load_u16(mk[0], mo[0], mask_base + (int64_t)pos * 2);
                load_u16(mk[1], mo[1], mask_base + (int64_t)pos * 2);
            }
        };
        auto request_v = [&](VBlock& vb, int64_t boff) {
            const char* bv = cache_v + boff;
            const char* sv = scale_v + (boff >> 3) * 2;
#pragma unroll
            for (int j = 0; j < kTB; ++j) {
                load_b128<GP == 1>(vb.q8[j], vo[j], bv);
                load_b32<false>(vb.sc[j], vo_sc[j], sv);
            }
        };

        KBlock ka, kb;
        VBlock va, vb;
        uint32_t mka[2] = {0, 0}, mkb[2] = {0, 0}; // the blocks' mask values (halves)
        int pos = pa32;
        if (nb == 1 && tail_partial) clamp_offsets(pos);
        request_k(ka, mka, pos);
        request_v(va, ka.boff);
        // the second block's K travels together with the first block: the loop's first iteration finds it requested
        // (a piece would otherwise pay a second memory latency before its second block)
        const int npos_first = pos + (nb > 1 ? BLK : 0);
        if (tail_partial && nb == 2) clamp_offsets(npos_first);
        request_k(kb, mkb, npos_first);

        // ---- A operands: this lane supplies row t4 = query head t4, its chunk's 16 channels ----
        half4_t qa[4];
        f32x4 qbias0, qbias1; // accumulator start per scale group: row g = -1152 * sum of head g's 8 channels
        {
            const bool on = g_first + t4 < G;
            const int h = kvh * G + (on ? g_first + t4 : 0);
            const u32x4* qp = (const u32x4*)((const half_t*)a.query + (int64_t)b * a.query_stride_s + (int64_t)h * D + ch0);
            u32x4 lo = qp[0], hi = qp[1];
            if (!on) { lo = u32x4{0, 0, 0, 0}; hi = lo; }
            qa[0] = bitcast<half4_t>(u32x2_t{lo[0], lo[1]});
            qa[1] = bitcast<half4_t>(u32x2_t{lo[2], lo[3]});
            qa[2] = bitcast<half4_t>(u32x2_t{hi[0], hi[1]});
            qa[3] = bitcast<half4_t>(u32x2_t{hi[2], hi[3]});
            float s0 = 0.f, s1 = 0.f;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                s0 += (float)qa[0][i] + (float)qa[1][i];
                s1 += (float)qa[2][i] + (float)qa[3][i];
            }
            s0 *= -1152.f;
            s1 *= -1152.f;
            qbias0 = f32x4{quad_lane<0>(s0), quad_lane<1>(s0), quad_lane<2>(s0), quad_lane<3>(s0)};
            qbias1 = f32x4{quad_lane<0>(s1), quad_lane<1>(s1), quad_lane<2>(s1), quad_lane<3>(s1)};
        }

        // online-softmax state: m_run / l_run for head g_own only (l_run over this lane's own logits);
        // acc[s] belongs to head g_first + (g_own ^ s)
        float m_run = kNegBig, l_run = 0.f;
        float acc[NS][16];
#pragma unroll
        for (int s = 0; s < NS; ++s)
#pragma unroll
            for (int c = 0; c < 16; ++c) acc[s][c] = 0.f;

        float prob[NS][kTB]; // [slot][step]: probabilities of this lane's own tokens
        // loads in flight when a block's logits start: its own, the V block before it and the next K block;
        // a K block has two more requests with the mask
        constexpr int kMoreK = MASK ? 4 : 0, kMoreV = MASK ? 2 : 0;
        // last: the piece's last block, behind which nothing but its own V block has been requested: one wait for the
        // whole K block then, since the counts below take a further K block's requests for granted (wave-uniform)
        auto logits_softmax = [&](KBlock& kx, uint32_t (&mk)[2], bool beyond_piece, bool last) { // beyond_piece: the block reaches past the piece (wave-uniform)
            if (last) {
                wait_block<8>(kx.q8, kx.sc);
                if (MASK) wait_loads<8>(mk[0], mk[1]);
            }
            float part[4][kTB]; // [head][step], over this lane's 16 channels, log2 units
#pragma unroll
            for (int j = 0; j < kTB; ++j) {
                if (j == 0) wait_loads<22 + kMoreK>(kx.q8[0], kx.sc[0]);
                if (j == 1) wait_loads<20 + kMoreK>(kx.q8[1], kx.sc[1]);
                if (j == 2) wait_loads<18 + kMoreK>(kx.q8[2], kx.sc[2]);
                if (j == 3) wait_loads<16 + kMoreK>(kx.q8[3], kx.sc[3]);
                f32x4 d0 = qbias0, d1 = qbias1;
#pragma unroll
                for (int w = 0; w < 4; ++w) {
                    const uint32_t f = kx.q8[j][w] ^ kFlipSigns;
                    const half4_t kh = bitcast<half4_t>(u32x2_t{__builtin_amdgcn_perm(kExpBytes, f, 0x04010400u),
                                                                __builtin_amdgcn_perm(kExpBytes, f, 0x04030402u)}); // 1152 + x
                    if (w < 2) d0 = __builtin_amdgcn_mfma_f32_4x4x4f16(qa[w], kh, d0, 0, 0, 0);
                    else d1 = __builtin_amdgcn_mfma_f32_4x4x4f16(qa[w], kh, d1, 0, 0, 0);
                }
                const half2_t sc = bitcast<half2_t>(kx.sc[j]);
                const float s0 = (float)sc.x, s1 = (float)sc.y; // the logit scale is applied to the two complete logits below
#pragma unroll
                for (int g = 0; g < 4; ++g) part[g][j] = __builtin_fmaf(d1[g], s1, d0[g] * s0);
            }
            if constexpr (H64) {
                // four chunk lanes: after the two folds a lane holds the complete logits of head g_own for all four
                // steps of its own tokens; nothing crosses the rows, whose lanes are separate token streams
                float l[kTB];
                float mx = kNegBig;
#pragma unroll
                for (int j = 0; j < kTB; ++j) {
                    const float ra0 = fold_xor4(part[0][j], part[2][j]);
                    const float ra1 = fold_xor4(part[1][j], part[3][j]);
                    l[j] = fold_xor8(ra0, ra1) * logit_scale;
                    if (beyond_piece) l[j] = kx.pos + 4 * j + tok0 < pe32 ? l[j] : -INFINITY;
                    mx = fmaxf(mx, l[j]);
                }
                const float m_new = fmaxf(m_run, mx);
                const bool moved = m_new > m_run;
                float p[kTB];
#pragma unroll
                for (int j = 0; j < kTB; ++j) p[j] = __builtin_amdgcn_exp2f(l[j] - m_new);
                if (__builtin_amdgcn_ballot_w64(moved) != 0) { // wave-uniform and rare: a running max moved
                    float al[4];
                    al[0] = __builtin_amdgcn_exp2f(m_run - m_new);
                    l_run *= al[0];
                    if constexpr (ONE) {
                        al[0] = from_head0_lane(al[0]);
                    } else {
                        al[1] = dpp_f32<kDppRor8>(al[0]);
                        al[2] = lane_xor4(al[0]);
                        al[3] = lane_xor4(al[1]);
                    }
#pragma unroll
                    for (int s = 0; s < NS; ++s)
#pragma unroll
                        for (int c = 0; c < 16; ++c) acc[s][c] *= al[s];
                }
                m_run = m_new;
                l_run += (p[0] + p[1]) + (p[2] + p[3]);
                if constexpr (ONE) {
#pragma unroll
                    for (int j = 0; j < kTB; ++j) prob[0][j] = from_head0_lane(p[j]);
                } else {
                    // all-gather of the heads over lane bits 3 and 2
#pragma unroll
                    for (int j = 0; j < kTB; ++j) {
                        prob[0][j] = p[j];
                        prob[1][j] = dpp_f32<kDppRor8>(p[j]);
                    }
#pragma unroll
                    for (int j = 0; j < kTB; ++j) {
                        prob[2][j] = lane_xor4(prob[0][j]);
                        prob[3][j] = lane_xor4(prob[1][j]);
                    }
                }
                return;
            }
            // reduce-scatter over the eight chunk lanes: lane bit 2 keeps heads {0,1} or {2,3}, bit 3 keeps
            // one of the pair, the row pair keeps steps {0,2} or {1,3}
            float l0, l1; // complete logits of head g_own: steps row_odd and 2 + row_odd
            {
                float rb[kTB];
#pragma unroll
                for (int j = 0; j < kTB; ++j) {
                    const float ra0 = fold_xor4(part[0][j], part[2][j]);
                    const float ra1 = fold_xor4(part[1][j], part[3][j]);
                    rb[j] = fold_xor8(ra0, ra1);
                }
                swap_rows(rb[0], rb[1]);
                swap_rows(rb[2], rb[3]);
                l0 = rb[0] + rb[1];
                l1 = rb[2] + rb[3];
                if (KPW == 1) { // the other half of the channels
                    l0 = sum_halves(l0);
                    l1 = sum_halves(l1);
                }
                l0 *= logit_scale;
                l1 *= logit_scale;
            }
            if (MASK) { // the block's two mask requests follow its eight cache requests
                wait_loads<18>(mk[0], mk[1]);
                l0 += (float)bitcast<half2_t>(mk[0]).x * kLog2e;
                l1 += (float)bitcast<half2_t>(mk[1]).x * kLog2e;
            }
            if (beyond_piece) { // only the last block of a piece
                const int tk = kx.pos + 4 * row_odd + t4;
                l0 = tk < pe32 ? l0 : -INFINITY;
                l1 = tk + 8 < pe32 ? l1 : -INFINITY;
            }
            // block max of the head: both lanes of the row pair
            float mx = fmaxf(l0, l1), my = mx;
            swap_rows(mx, my);
            const float m_new = fmaxf(m_run, fmaxf(mx, my));
            const bool moved = m_new > m_run;
            float p0 = __builtin_amdgcn_exp2f(l0 - m_new);
            float p1 = __builtin_amdgcn_exp2f(l1 - m_new);
            if (__builtin_amdgcn_ballot_w64(moved) != 0) { // wave-uniform and rare: a running max moved
                float al[4];
                al[0] = __builtin_amdgcn_exp2f(m_run - m_new);
                l_run *= al[0];
                if constexpr (ONE) {
                    al[0] = from_head0_lane(al[0]);
                } else {
                    al[1] = dpp_f32<kDppRor8>(al[0]);
                    al[2] = lane_xor4(al[0]);
                    al[3] = lane_xor4(al[1]);
                }
#pragma unroll
                for (int s = 0; s < NS; ++s)
#pragma unroll
                    for (int c = 0; c < 16; ++c) acc[s][c] *= al[s];
            }
            m_run = m_new;
            l_run += p0 + p1;
            // all-gather: steps over the row pair, heads over lane bits 3 and 2
            float q0 = p0, q1 = p1;
            swap_rows(p0, q0); // p0 = step 0, q0 = step 1
            swap_rows(p1, q1); // p1 = step 2, q1 = step 3
            if constexpr (ONE) {
                prob[0][0] = from_head0_lane(p0);
                prob[0][1] = from_head0_lane(q0);
                prob[0][2] = from_head0_lane(p1);
                prob[0][3] = from_head0_lane(q1);
            } else {
                prob[0][0] = p0; prob[0][1] = q0; prob[0][2] = p1; prob[0][3] = q1;
#pragma unroll
                for (int j = 0; j < kTB; ++j) prob[1][j] = dpp_f32<kDppRor8>(prob[0][j]);
#pragma unroll
                for (int j = 0; j < kTB; ++j) {
                    prob[2][j] = lane_xor4(prob[0][j]);
                    prob[3][j] = lane_xor4(prob[1][j]);
                }
            }
        };

        auto accumulate_pv = [&](VBlock& vx, bool last) { // last: nothing requested behind this V block
            if (last) wait_block<0>(vx.q8, vx.sc);
#pragma unroll
            for (int j = 0; j < kTB; ++j) {
                if (j == 0) wait_loads<22 + kMoreV>(vx.q8[0], vx.sc[0]);
                if (j == 1) wait_loads<20 + kMoreV>(vx.q8[1], vx.sc[1]);
                if (j == 2) wait_loads<18 + kMoreV>(vx.q8[2], vx.sc[2]);
                if (j == 3) wait_loads<16 + kMoreV>(vx.q8[3], vx.sc[3]);
                float x[16];
#pragma unroll
                for (int w = 0; w < 4; ++w) {
                    x[4 * w + 0] = byte_to_f32<0>(vx.q8[j][w]);
                    x[4 * w + 1] = byte_to_f32<1>(vx.q8[j][w]);
                    x[4 * w + 2] = byte_to_f32<2>(vx.q8[j][w]);
                    x[4 * w + 3] = byte_to_f32<3>(vx.q8[j][w]);
                }
                const half2_t sc = bitcast<half2_t>(vx.sc[j]);
                const float sv0 = (float)sc.x, sv1 = (float)sc.y;
#pragma unroll
                for (int s = 0; s < NS; ++s) {
                    const float w0 = prob[s][j] * sv0, w1 = prob[s][j] * sv1;
#pragma unroll
                    for (int c = 0; c < 8; ++c) {
                        acc[s][c] = __builtin_fmaf(w0, x[c], acc[s][c]);
                        acc[s][8 + c] = __builtin_fmaf(w1, x[8 + c], acc[s][8 + c]);
                    }
                }
            }
        };

        // An empty statement that every accumulator passes through at the end of a block.  Without it the
        // register allocator keeps the accumulators of the two unrolled blocks in different registers and
        // copies all 64 of them twice per loop iteration (8 % of the loop's instructions).
        auto pin_acc = [&]() {
#pragma unroll
            for (int s = 0; s < NS; ++s)
#pragma unroll
                for (int c = 0; c < 16; ++c) asm volatile("" : "+v"(acc[s][c]));
        };

        // software pipeline as in decode_attn.hip: K of block i+1 is requested before the logits of
        // block i, V of block i+1 before the PV of block i; the last block re-requests itself
        drain_loads(ka.q8, ka.sc);
        drain_loads(va.q8, va.sc);
        if (MASK) wait_loads<0>(mka[0], mka[1]);
        for (int i = 0;;) {
            // With two sets of waves on the same kv heads, a barrier per pair of blocks keeps the sets within a
            // block of each other, so that the second set's requests find the lines in the cache levels
            // (every wave of the workgroup runs the same number of blocks).
            if (GP > 1) __syncthreads();
            // The piece's last block requests nothing: what it requested would only be waited for before the merge, a
            // memory latency per piece for nothing.
            bool last = i + 1 == nb;
            int npos = npos_first;
            if (i > 0 && !last) {
                npos = pos + BLK;
                if (tail_partial && i + 2 == nb) clamp_offsets(npos);
                request_k(kb, mkb, npos);
            }
            logits_softmax(ka, mka, tail_partial && last, last);
            if (!last) request_v(vb, kb.boff);
            accumulate_pv(va, last);
            pin_acc();
            pos = npos;
            if (++i == nb) break;
            last = i + 1 == nb;
            if (!last) {
                npos = pos + BLK;
                if (tail_partial && i + 2 == nb) clamp_offsets(npos);
                request_k(ka, mka, npos);
            }
            logits_softmax(kb, mkb, tail_partial && last, last);
            if (!last) request_v(va, ka.boff);
            accumulate_pv(vb, last);
            pin_acc();
            pos = npos;
            if (++i == nb) break;
        }
        drain_loads(ka.q8, ka.sc);
        drain_loads(kb.q8, kb.sc);
        drain_loads(va.q8, va.sc);
        drain_loads(vb.q8, vb.sc);
        if (MASK) {
            wait_loads<0>(mka[0], mka[1]);
            wait_loads<0>(mkb[0], mkb[1]);
        }

        // ---- end of the piece: exp-sum of the head over the row pair, (max, sum) of the four slots,
        // then the four token streams of the quad are merged ----
        if constexpr (!H64) {
            float lx = l_run, ly = l_run;
            swap_rows(lx, ly);
            l_run = lx + ly;
        }
        // head_dim 64: the two rows of a half-wave are two more token streams of the same heads and channels; their
        // (max, sum, accumulators) are merged with those of the quad below (the swap hands a lane its own value and
        // that of lane ^ 16, so a sum or a maximum of the two results needs no select)
        auto across_rows_max = [&](float v) {
            if constexpr (!H64) return v;
            float x = v, y = v;
            swap_rows(x, y);
            return fmaxf(x, y);
        };
        auto across_rows_sum = [&](float v) {
            if constexpr (!H64) return v;
            float x = v, y = v;
            swap_rows(x, y);
            return x + y;
        };
        float ms[4], lsum[4];
        ms[0] = m_run;
        lsum[0] = l_run;
        if constexpr (ONE) { // head 0's state, which the lanes of the absent heads take from its chunk lane
            ms[0] = from_head0_lane(ms[0]);
            lsum[0] = from_head0_lane(lsum[0]);
        } else {
            ms[1] = dpp_f32<kDppRor8>(ms[0]);
            lsum[1] = dpp_f32<kDppRor8>(lsum[0]);
            ms[2] = lane_xor4(ms[0]);
            ms[3] = lane_xor4(ms[1]);
            lsum[2] = lane_xor4(lsum[0]);
            lsum[3] = lane_xor4(lsum[1]);
        }

        const bool whole = (pa == 0) && (pe == len);
        const int64_t piece = (int64_t)blockIdx.x + b;
#pragma unroll
        for (int s = 0; s < NS; ++s) {
            float M = fmaxf(ms[s], dpp_f32<kDppXor1>(ms[s]));
            M = fmaxf(M, dpp_f32<kDppXor2>(M));
            M = across_rows_max(M);
            const float w = __builtin_amdgcn_exp2f(ms[s] - M);
            float L = lsum[s] * w;
            L += dpp_f32<kDppXor1>(L);
            L += dpp_f32<kDppXor2>(L);
            L = across_rows_sum(L);
            const float inv = L > 0.f ? 1.f / L : 0.f;
            float o[16];
#pragma unroll
            for (int c = 0; c < 16; ++c) {
                float v = acc[s][c] * w;
                v += dpp_f32<kDppXor1>(v);
                v += dpp_f32<kDppXor2>(v);
                o[c] = across_rows_sum(v) * inv;
            }
            const int g = ONE ? 0 : g_first + (g_own ^ s);
            if (t4 == 0 && (!H64 || row_odd == 0) && g < G && head_on) {
                const int h = kvh * G + g;
                if (whole) {
                    typedef half_t half8_t __attribute__((ext_vector_type(8)));
                    half_t* out = (half_t*)a.output + (int64_t)b * a.output_stride_s + (int64_t)h * D + ch0;
                    half8_t v0, v1;
#pragma unroll
                    for (int c = 0; c < 8; ++c) {
                        v0[c] = (half_t)o[c];
                        v1[c] = (half_t)o[8 + c];
                    }
                    *(half8_t*)out = v0;
                    *(half8_t*)(out + 8) = v1;
                } else {
                    float* out = a.partial_out + (piece * a.num_heads + h) * D + ch0;
#pragma unroll
                    for (int c = 0; c < 16; c += 4) *(f32x4*)(out + c) = f32x4{o[c], o[c + 1], o[c + 2], o[c + 3]};
                    if (chunk == 0) {
                        a.partial_ml[(piece * a.num_heads + h) * 2 + 0] = M;
                        a.partial_ml[(piece * a.num_heads + h) * 2 + 1] = L;
                    }
                }
            }
        }
    }
}

// One or two query heads per kv head leave rows of the 4x4x4 products and three quarters or half of the PV
// arithmetic unused, but this kernel's row loads take the non-temporal hint, which the general kernel's cannot.
// Which shapes come here is decided in decode_select.cpp.
template <int WP, int HD>
static void launch_decode_quad_wp(const DecodeLaunch& a, hipStream_t stream)
{
    constexpr int KPW = HD == 256 ? 1 : 2;
    const dim3 grid((unsigned)a.ranges, (unsigned)((a.num_kv_heads + KPW * WP - 1) / (KPW * WP)), 1);
    const bool paged = a.cache_mode == 1, mask = a.attn_mask != nullptr;
    const bool one = a.num_kv_repeats == 1; // MHA: a single head slot per lane
    if (paged) {
        if (mask) hipLaunchKernelGGL((decode_attention_quad_kernel<true, 1, WP, true, HD>), grid, dim3(kWave * WP), 0, stream, a);
        else if (one) hipLaunchKernelGGL((decode_attention_quad_kernel<true, 1, WP, false, HD, 1>), grid, dim3(kWave * WP), 0, stream, a);
        else hipLaunchKernelGGL((decode_attention_quad_kernel<true, 1, WP, false, HD>), grid, dim3(kWave * WP), 0, stream, a);
    } else {
        if (mask) hipLaunchKernelGGL((decode_attention_quad_kernel<false, 1, WP, true, HD>), grid, dim3(kWave * WP), 0, stream, a);
        else if (one) hipLaunchKernelGGL((decode_attention_quad_kernel<false, 1, WP, false, HD, 1>), grid, dim3(kWave * WP), 0, stream, a);
        else hipLaunchKernelGGL((decode_attention_quad_kernel<false, 1, WP, false, HD>), grid, dim3(kWave * WP), 0, stream, a);
    }
}

template <int WP, int HD>
static void launch_decode_quad_two_sets(const DecodeLaunch& a, hipStream_t stream)
{
    constexpr int KPW = HD == 256 ? 1 : 2;
    const dim3 grid((unsigned)a.ranges, (unsigned)(a.num_kv_heads / (KPW * WP)), 1);
    if (a.cache_mode == 1) hipLaunchKernelGGL((decode_attention_quad_kernel<true, 2, WP, false, HD>), grid, dim3(2 * WP * kWave), 0, stream, a);
    else hipLaunchKernelGGL((decode_attention_quad_kernel<false, 2, WP, false, HD>), grid, dim3(2 * WP * kWave), 0, stream, a);
}

void launch_decode_quad(const DecodeLaunch& a, hipStream_t stream)
{
    const int waves = a.kv_heads_per_group / (a.head_dim == 256 ? 1 : 2);
    if (a.num_kv_repeats > 4) { // two sets of waves: the second takes query heads 4-7 of the same kv heads
        if (a.head_dim == 256) { // a wave per kv head
            switch (waves) {
            case 4: launch_decode_quad_two_sets<4, 256>(a, stream); break;
            case 2: launch_decode_quad_two_sets<2, 256>(a, stream); break;
            default: launch_decode_quad_two_sets<1, 256>(a, stream); break;
            }
        } else {
            launch_decode_quad_two_sets<4, 128>(a, stream); // eight kv heads
        }
        return;
    }
    if (a.head_dim == 64) { // no mask form: decode_quad_launch_ok sends masked steps to the general kernel
        const dim3 grid((unsigned)a.ranges, (unsigned)((a.num_kv_heads + 2 * waves - 1) / (2 * waves)), 1);
        const bool paged = a.cache_mode == 1;
        switch (waves) {
        case 4:
            if (paged) hipLaunchKernelGGL((decode_attention_quad_kernel<true, 1, 4, false, 64>), grid, dim3(kWave * 4), 0, stream, a);
            else hipLaunchKernelGGL((decode_attention_quad_kernel<false, 1, 4, false, 64>), grid, dim3(kWave * 4), 0, stream, a);
            break;
        case 2:
            if (paged) hipLaunchKernelGGL((decode_attention_quad_kernel<true, 1, 2, false, 64>), grid, dim3(kWave * 2), 0, stream, a);
            else hipLaunchKernelGGL((decode_attention_quad_kernel<false, 1, 2, false, 64>), grid, dim3(kWave * 2), 0, stream, a);
            break;
        default:
            if (paged) hipLaunchKernelGGL((decode_attention_quad_kernel<true, 1, 1, false, 64>), grid, dim3(kWave), 0, stream, a);
            else hipLaunchKernelGGL((decode_attention_quad_kernel<false, 1, 1, false, 64>), grid, dim3(kWave), 0, stream, a);
            break;
        }
        return;
    }
    if (a.head_dim == 256) {
        switch (waves) {
        case 4: launch_decode_quad_wp<4, 256>(a, stream); break;
        case 2: launch_decode_quad_wp<2, 256>(a, stream); break;
        default: launch_decode_quad_wp<1, 256>(a, stream); break;
        }
    } else {
        switch (waves) {
        case 4: launch_decode_quad_wp<4, 128>(a, stream); break;
        case 2: launch_decode_quad_wp<2, 128>(a, stream); break;
        default: launch_decode_quad_wp<1, 128>(a, stream); break;
        }
    }
}

} // namespace pmxhip
