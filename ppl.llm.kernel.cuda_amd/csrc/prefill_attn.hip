// Multi-query-token (chunked prefill) attention over the int8 group-8 KV cache
// for gfx950, on MFMA.
//
// Semantics follow the reference's prefill stage
// (src/ppl/kernel/llm/cuda/pmx/multi_head_cache_attention/kernel.cu:2127-2179, which
// calls flash_attn2_paged_fmha): query rows seqstarts[b]..seqstarts[b+1], kv length
// kvstarts[b+1]-kvstarts[b], K/V from the int8 cache through cachestarts, dequantised
// as fp16(int8) * fp16(scale) (flash_attn2/src/utils.h:397-436), causal mask aligned
// bottom-right: row i sees columns < i + 1 + kvlen - qlen (flash_attn2/src/mask.h:186).
//
// Decomposition (this file's own):
//   * one workgroup (8 waves, two per SIMD) = one kv head of one sequence x a tile
//     of query positions x ALL query heads of that kv head.  The (position, head)
//     pairs are the 256 "columns" of the tile, 32 per wave, so a dequantised K/V
//     tile is shared by every query head of the group.
//   * K/V tiles of 64 tokens are dequantised int8 -> fp16 into LDS once per
//     workgroup, into one of two buffers: while tile i is multiplied, tile i+1 is
//     dequantised into the other buffer and the raw bytes of tile i+2 travel from
//     memory into registers.  One barrier per tile.
//   * S^T = K Q^T (tokens are MFMA rows, columns stay columns): a lane then owns
//     one column, so the softmax max/sum are register-local apart from one
//     exchange between the two half-waves, and the S^T accumulator layout is
//     already the B-operand layout of O^T = V^T P^T -- no shuffle between the
//     two MFMA stages.  V is stored transposed in LDS with tokens permuted to
//     match that layout.
//   * v_mfma_f32_32x32x16_f16, fp32 accumulate, base-2 online softmax.
#include "device_common.h"
#include "launch_params.h"

namespace pmxhip {

namespace {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int kPrefillThreads = 512;
constexpr int kBN = 64;        // kv tokens per tile
constexpr int kCols = 256;     // (position, head) columns per workgroup, 32 per wave
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kNegBig = -1.0e30f;
constexpr float kPShift = 14.0f;

// position of token offset o (0..15) inside its 16-token group of the transposed V tile:
// token bits (a, h, r1, r0) -> position bits (h, a, r1, r0)
__device__ __forceinline__ int vt_pos16(int o) { return ((o & 4) << 1) | ((o & 8) >> 1) | (o & 3); }

// sum over the wave of small non-negative integers, one ballot per bit (every lane of the wave must be here)
__device__ __forceinline__ int wave_sum_small(int v)
{
    int sum = 0;
    for (int bit = 0; __builtin_amdgcn_ballot_w64((v >> bit) != 0) != 0; ++bit)
        sum += __builtin_popcountll(__builtin_amdgcn_ballot_w64(((v >> bit) & 1) != 0)) << bit;
    return sum;
}

// Which query tile a workgroup takes.  The tiles of a ragged batch cost very different amounts (a tile walks the kv
// tokens up to its last query row: prior context + rows so far), a CU holds one workgroup, and workgroups start in
// the order of their numbers, so the order decides how long the last CUs run alone: with the dear tiles first the
// cheap ones fill the gaps at the end.  Tile t of sequence s gets the level t + ceil(prior_s / ppw) (its cost in
// units of ppw tokens) and item i of the launch is the i-th tile in the order of falling level (sequences in
// index order inside a level).  Every wave finds its tile by itself from seqstarts/kvstarts: a lane holds the
// level interval [lo, lo + n) of up to kPickSlots sequences, the number of tiles at or above a level is a sum over
// the lanes, and the item's level follows by bisection.  Beyond 64 * kPickSlots sequences the order is the plain
// one (last tiles first, sequences in index order).  Returns false for an item beyond the batch's tiles.
constexpr int kPickSlots = 16;
__device__ __forceinline__ bool pick_query_tile(const PrefillLaunch& a, int ppw, int item, int lane, int& b_out, int& tile_out)
{
    const int nseq = (int)a.prefill_batches;
    if (nseq > 64 * kPickSlots) {
        const int tiles_max = (int)((a.max_seqlen + ppw - 1) / ppw);
        const int y = item / nseq;
        b_out = item - y * nseq;
        tile_out = tiles_max - 1 - y;
        return y < tiles_max;
    }
    const int kmax = (nseq + 63) >> 6;
    int lo[kPickSlots], n[kPickSlots];
    int hi_lane = 0;
#pragma unroll
    for (int k = 0; k < kPickSlots; ++k) {
        lo[k] = 0;
        n[k] = 0;
        if (k < kmax) {
            const int s = 64 * k + lane;
            if (s < nseq) {
                const int qlen = (int)(a.seqstarts[s + 1] - a.seqstarts[s]);
                const int kvlen = (int)(a.kvstarts[s + 1] - a.kvstarts[s]);
                int prior = a.is_causal ? kvlen - qlen : kvlen;
                prior = prior > 0 ? prior : 0;
                lo[k] = (prior + ppw - 1) / ppw;
                n[k] = qlen > 0 ? (qlen + ppw - 1) / ppw : 0;
                hi_lane = hi_lane > lo[k] + n[k] ? hi_lane : lo[k] + n[k];
            }
        }
    }
    // tiles at or above level l
    auto count_from = [&](int l) {
        int c = 0;
#pragma unroll
        for (int k = 0; k < kPickSlots; ++k)
            if (k < kmax) {
                const int from = l > lo[k] ? l : lo[k];
                const int d = lo[k] + n[k] - from;
                c += d > 0 ? d : 0;
            }
        return wave_sum_small(c);
    };
    if (item >= count_from(0)) return false;
    // the largest level end of the wave, bit by bit
    int top = 0;
    for (int bit = 24; bit >= 0; --bit)
        if (__builtin_amdgcn_ballot_w64(hi_lane >= (top | (1 << bit))) != 0) top |= 1 << bit;
    int below = 0, above = top; // count_from(below) > item >= count_from(above)
    while (above - below > 1) {
        const int mid = (below + above) >> 1;
        if (count_from(mid) > item) below = mid;
        else above = mid;
    }
    const int level = below;
    int r = item - count_from(level + 1); // index among the sequences that have a tile at this level
#pragma unroll
    for (int k = 0; k < kPickSlots; ++k)
        if (k < kmax) {
            const bool has = lo[k] <= level && level < lo[k] + n[k];
            const uint64_t mask = __builtin_amdgcn_ballot_w64(has);
            const int cnt = __builtin_popcountll(mask);
            if (r < cnt) {
                const int before = __builtin_popcountll(mask & ((1ull << lane) - 1ull));
                const uint64_t sel = __builtin_amdgcn_ballot_w64(has && before == r);
                const int src = __builtin_ctzll(sel);
                b_out = 64 * k + src;
                tile_out = level - __builtin_amdgcn_readlane(lo[k], src);
                return true;
            }
            r -= cnt;
        }
    return false;
}

} // namespace

// SRC: where K/V come from: 0 = int8 cache in 128-token pages, 1 = int8 cache in contiguous runs,
// 2 = the step's fp16 current_key/current_value rows.  EXTRA: additive attn_mask and/or alibi slopes.
template <int D, int SRC, bool EXTRA>
__global__ __launch_bounds__(kPrefillThreads, 2) void prefill_attention_kernel(const PrefillLaunch a)
{
    constexpr bool PAGED = SRC == 0;
    constexpr bool KV16 = SRC == 2;
    constexpr int KSTEPS = D / 16;          // MFMA k-steps over channels for S
    constexpr int CB = D / 32;              // 32-channel blocks of O^T
    constexpr int GPT = D / 8;              // quantisation groups per token row
    constexpr int K_STRIDE = D + 8;         // halves per K row in LDS (+16 B: conflict-free b128 reads)
    constexpr int V_STRIDE = kBN + 8;       // halves per V^T row in LDS
    constexpr int K_UNITS = kBN * GPT / kPrefillThreads;  // (token, group) units per thread
    constexpr int V_THREADS = (kBN / 4) * GPT;            // threads with a (token quad, group) unit

    // K is kept as an unevaluated sum hi + lo of two halves: hi = fp16(int8 * scale) and
    // lo = the rounding error of that product (exact, from one fused multiply-add), so that
    // q.k carries no fp16 rounding of the dequantised key.  With a single rounded copy a
    // 2^-12 relative error on |q_c k_c| ~ 1e3 (outlier channels) moves logits by ~1e-2.
    // V and the probabilities are split the same way (V^ = hi + lo from the same multiply-add
    // trick, p = hi + lo), and O accumulates hi*hi + lo*hi + hi*lo: at |v| ~ 40 a single fp16
    // rounding of either factor already costs ~1e-2 absolute where contributions cancel.
    extern __shared__ __attribute__((aligned(16))) char smem_raw[];
    // two tile buffers; a buffer holds K (hi, lo) row-major and V (hi, lo) transposed
    // (fp16 K/V need no low parts: the tiles are the values themselves)
    constexpr int TILE_HALVES = (KV16 ? 1 : 2) * (kBN * K_STRIDE + D * V_STRIDE);
    half_t* const smem = (half_t*)smem_raw;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int hh = lane >> 5;   // half-wave
    const int l32 = lane & 31;

    // grid: workgroup = (item, kv head), kv head fastest; item i is the i-th query tile of the batch in the order
    // of falling cost (pick_query_tile), and workgroups start in the order of their numbers
    const int G = (int)(a.num_heads / a.num_kv_heads);
    const int ppw = kCols / G > 0 ? kCols / G : 1; // query positions per workgroup
    const int item = blockIdx.x / (int)a.num_kv_heads;
    const int kvh = blockIdx.x - item * (int)a.num_kv_heads;
    int b_pick = 0, tile_pick = 0;
    if (!pick_query_tile(a, ppw, item, lane, b_pick, tile_pick)) return;
    const int b = __builtin_amdgcn_readfirstlane(b_pick);
    const int64_t q_row0 = a.seqstarts[b];
    const int qlen = (int)(a.seqstarts[b + 1] - q_row0);
    const int kvlen = (int)(a.kvstarts[b + 1] - a.kvstarts[b]);
    const int p0 = __builtin_amdgcn_readfirstlane(tile_pick) * ppw;
    if (p0 < 0 || p0 >= qlen) return;

    // ---- this lane's column ----
    const int col = wave * 32 + l32;
    const int pos = p0 + col / G;
    const int g = col % G;
    const bool col_on = (col < ppw * G) && (pos < qlen);
    const int pos_c = pos < qlen ? pos : qlen - 1;
    const int h = kvh * G + (col < ppw * G ? g : 0);
    int lim = kvlen;                                   // this column attends tokens [0, lim)
    if (a.is_causal) {
        lim = pos_c + 1 + kvlen - qlen;
        lim = lim < 0 ? 0 : (lim > kvlen ? kvlen : lim);
    }
    if (!col_on) lim = 0;
    // tokens the workgroup must walk: the largest limit of its columns
    int last_pos = p0 + ppw - 1;
    if (last_pos > qlen - 1) last_pos = qlen - 1;
    int wg_lim = kvlen;
    if (a.is_causal) {
        wg_lim = last_pos + 1 + kvlen - qlen;
        wg_lim = wg_lim < 0 ? 0 : (wg_lim > kvlen ? kvlen : wg_lim);
    }
    const int n_tiles = (wg_lim + kBN - 1) / kBN;

    // ---- Q fragments: B operand of S^T = K Q^T; lane holds Q[col][16 s + 8 hh .. +8] ----
    f16x8 qf[KSTEPS];
    {
        const half_t* qp = (const half_t*)a.query + (q_row0 + pos_c) * a.query_stride_s + (int64_t)h * D + 8 * hh;
#pragma unroll
        for (int s = 0; s < KSTEPS; ++s) qf[s] = *(const f16x8*)(qp + 16 * s);
    }

    f32x16 o_acc[CB];
#pragma unroll
    for (int cb = 0; cb < CB; ++cb)
#pragma unroll
        for (int i = 0; i < 16; ++i) o_acc[cb][i] = 0.f;
    float m_run = kNegBig, l_run = 0.f;
    const float sm_scale = a.attn_scale * kLog2e;
    // element (head, absolute query row, absolute kv column) of the additive mask; kvstarts holds absolute columns
    const half_t* mask_row = nullptr;
    float slope = 0.f;
    if (EXTRA) {
        if (a.attn_mask)
            mask_row = (const half_t*)a.attn_mask + (int64_t)h * a.mask_stride_h + (q_row0 + pos_c) * a.mask_stride_s + a.kvstarts[b];
        if (a.alibi_slopes) slope = a.alibi_slopes[h];
    }

    // ---- global -> register staging of one tile's raw bytes ----
    const int8_t* __restrict__ cache = (const int8_t*)a.cache;
    const half_t* __restrict__ scale = (const half_t*)a.scale;
    const int64_t head_off = a.layer_idx * a.cache_stride_l + (int64_t)kvh * a.cache_stride_h;
    const int64_t table_base = PAGED ? (int64_t)b * a.cachestarts_stride_b : (int64_t)b;

    const int k_g = tid % GPT;           // channel group of this thread's K units
    const int k_t0 = tid / GPT;          // first token; further units are kPrefillThreads / GPT tokens apart
    const int v_g = tid % GPT;
    const int v_q = (tid / GPT) % (kBN / 4); // token quad (tokens 4 v_q .. 4 v_q + 3)
    const int v_half = tid / V_THREADS;      // which four of the group's eight channels this thread transposes
    const bool v_on = (2 * V_THREADS == kPrefillThreads) || v_half < 2; // compile-time true when every thread has a unit

    u32x2 k_raw[K_UNITS];
    half_t k_sc[K_UNITS];
    u32x2 v_raw[4];
    half_t v_sc[4];
    u32x4 k16[K_UNITS], v16[4]; // fp16 source: 8 halves per unit

    // Addressing: a tile of 64 tokens starts at a multiple of 64, so it lies inside one page.  Its row
    // base is wave-uniform (scalar loads of the page table, read one tile ahead); the per-lane part
    // (token in tile, channel group) never changes and is computed once.
    const const_i64_ptr cachestarts = as_constant(a.cachestarts);
    auto tile_row = [&](int tile) -> int64_t {
        int t_base = tile * kBN;
        if (t_base > kvlen - 1) t_base = kvlen > 0 ? kvlen - 1 : 0;
        if (KV16) return q_row0 + t_base; // current_key row of kv token t = query row of the same position
        if (PAGED) return cachestarts[table_base + (t_base >> 7)] + (t_base & (kPage - 1));
        return cachestarts[table_base] + t_base;
    };
    const uint32_t stride_s32 = (uint32_t)a.cache_stride_s; // the host checks that a tile's span fits 32 bits
    constexpr int K_TSTEP = kPrefillThreads / GPT;           // tokens between a thread's K units
    uint32_t k_off[K_UNITS], v_off[4];
#pragma unroll
    for (int u = 0; u < K_UNITS; ++u) k_off[u] = (uint32_t)(k_t0 + u * K_TSTEP) * stride_s32 + 8 * k_g;
#pragma unroll
    for (int r = 0; r < 4; ++r) v_off[r] = (uint32_t)(4 * v_q + r) * stride_s32 + 8 * v_g;
    const int8_t* const cache_k = cache + head_off;
    const int8_t* const cache_v = cache_k + a.cache_stride_kv;
    const half_t* const scale_k = scale + (head_off >> 3);
    const half_t* const scale_v = scale_k + (a.cache_stride_kv >> 3);

    const uint32_t kstride16 = (uint32_t)a.key_stride_s, vstride16 = (uint32_t)a.value_stride_s;
    auto load_tile = [&](int tile, int64_t row) {
        if (KV16) {
            const half_t* bk = (const half_t*)a.current_key + row * a.key_stride_s + (int64_t)kvh * D;
            const half_t* bv = (const half_t*)a.current_value + row * a.value_stride_s + (int64_t)kvh * D;
            const int left = kvlen - 1 - tile * kBN;
#pragma unroll
            for (int u = 0; u < K_UNITS; ++u) {
                int t = k_t0 + u * K_TSTEP;
                t = t < left ? t : (left > 0 ? left : 0);
                k16[u] = *(const u32x4*)(bk + (uint32_t)t * kstride16 + 8 * k_g);
            }
            if (v_on) {
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    int t = 4 * v_q + r;
                    t = t < left ? t : (left > 0 ? left : 0);
                    v16[r] = *(const u32x4*)(bv + (uint32_t)t * vstride16 + 8 * v_g);
                }
            }
            return;
        }
        const int64_t boff = row * a.cache_stride_s;
        const int8_t* bk = cache_k + boff;
        const int8_t* bv = cache_v + boff;
        const half_t* sk = scale_k + (boff >> 3);
        const half_t* sv = scale_v + (boff >> 3);
        const int left = kvlen - 1 - tile * kBN; // offset of the sequence's last token inside this tile
        if (left >= kBN - 1) {
#pragma unroll
            for (int u = 0; u < K_UNITS; ++u) {
                k_raw[u] = *(const u32x2*)(bk + k_off[u]);
                k_sc[u] = sk[k_off[u] >> 3];
            }
            if (v_on) {
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    v_raw[r] = *(const u32x2*)(bv + v_off[r]);
                    v_sc[r] = sv[v_off[r] >> 3];
                }
            }
        } else { // last tile of the sequence: tokens beyond it re-read its last token (masked later)
#pragma unroll
            for (int u = 0; u < K_UNITS; ++u) {
                const int t = k_t0 + u * K_TSTEP;
                const uint32_t off = (uint32_t)(t < left ? t : (left > 0 ? left : 0)) * stride_s32 + 8 * k_g;
                k_raw[u] = *(const u32x2*)(bk + off);
                k_sc[u] = sk[off >> 3];
            }
            if (v_on) {
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int t = 4 * v_q + r;
                    const uint32_t off = (uint32_t)(t < left ? t : (left > 0 ? left : 0)) * stride_s32 + 8 * v_g;
                    v_raw[r] = *(const u32x2*)(bv + off);
                    v_sc[r] = sv[off >> 3];
                }
            }
        }
    };
    // One slice of the dequantise-and-store of a tile: slices [0, K_UNITS) are this thread's K units, slices
    // K_UNITS + [0, 4) its four V channels.  Sliced so that the work can be spread between the MFMAs of the
    // previous tile's products.
    constexpr int N_SLICES = K_UNITS + 4;
    auto store_slice = [&](int buf, int slice) {
        half_t* const sK = smem + buf * TILE_HALVES;
        half_t* const sKlo = sK + kBN * K_STRIDE;
        half_t* const sV = KV16 ? sKlo : sKlo + kBN * K_STRIDE;
        half_t* const sVlo = sV + D * V_STRIDE;
        if (KV16) {
#pragma unroll
            for (int u = 0; u < K_UNITS; ++u)
                if (slice == u) *(u32x4*)&sK[(k_t0 + u * K_TSTEP) * K_STRIDE + 8 * k_g] = k16[u];
            if (v_on) {
                const int grp = v_q >> 2;
                const int posv = 16 * grp + vt_pos16(4 * (v_q & 3));
#pragma unroll
                for (int e4 = 0; e4 < 4; ++e4) {
                    if (slice != K_UNITS + e4) continue;
                    const int e = 4 * v_half + ((e4 + v_g) & 3); // rotated channel order, as below
                    const uint32_t sel = (e & 1) ? 0x07060302u : 0x05040100u; // half (e & 1) of two words
                    const int w = e >> 1;
                    const uint32_t w0 = w == 0 ? v16[0][0] : (w == 1 ? v16[0][1] : (w == 2 ? v16[0][2] : v16[0][3]));
                    const uint32_t w1 = w == 0 ? v16[1][0] : (w == 1 ? v16[1][1] : (w == 2 ? v16[1][2] : v16[1][3]));
                    const uint32_t w2 = w == 0 ? v16[2][0] : (w == 1 ? v16[2][1] : (w == 2 ? v16[2][2] : v16[2][3]));
                    const uint32_t w3 = w == 0 ? v16[3][0] : (w == 1 ? v16[3][1] : (w == 2 ? v16[3][2] : v16[3][3]));
                    u32x2 out;
                    out[0] = __builtin_amdgcn_perm(w1, w0, sel);
                    out[1] = __builtin_amdgcn_perm(w3, w2, sel);
                    *(u32x2*)&sV[(8 * v_g + e) * V_STRIDE + posv] = out;
                }
            }
            return;
        }
        // K: 8 halves of one (token, group) -> one 128-bit LDS store
#pragma unroll
        for (int u = 0; u < K_UNITS; ++u) {
            if (slice != u) continue;
            const half2_t sc = {k_sc[u], k_sc[u]};
            const uint32_t f0 = k_raw[u][0] ^ kFlipSigns, f1 = k_raw[u][1] ^ kFlipSigns;
            const half2_t x0 = cvt_bytes01(f0), x1 = cvt_bytes23(f0), x2 = cvt_bytes01(f1), x3 = cvt_bytes23(f1);
            const half2_t h0 = x0 * sc, h1 = x1 * sc, h2 = x2 * sc, h3 = x3 * sc;
            u32x4 w, wl;
            w[0] = bitcast<uint32_t>(h0);
            w[1] = bitcast<uint32_t>(h1);
            w[2] = bitcast<uint32_t>(h2);
            w[3] = bitcast<uint32_t>(h3);
            wl[0] = bitcast<uint32_t>(__builtin_elementwise_fma(x0, sc, -h0));
            wl[1] = bitcast<uint32_t>(__builtin_elementwise_fma(x1, sc, -h1));
            wl[2] = bitcast<uint32_t>(__builtin_elementwise_fma(x2, sc, -h2));
            wl[3] = bitcast<uint32_t>(__builtin_elementwise_fma(x3, sc, -h3));
            const int t = k_t0 + u * (kPrefillThreads / GPT);
            *(u32x4*)&sK[t * K_STRIDE + 8 * k_g] = w;
            *(u32x4*)&sKlo[t * K_STRIDE + 8 * k_g] = wl;
        }
        // V: four tokens of one channel -> one 64-bit LDS store into the transposed tile
        if (v_on) {
            const half2_t s01 = {v_sc[0], v_sc[1]}, s23 = {v_sc[2], v_sc[3]};
            const int grp = v_q >> 2;
            const int posv = 16 * grp + vt_pos16(4 * (v_q & 3));
#pragma unroll
            for (int e4 = 0; e4 < 4; ++e4) {
                if (slice != K_UNITS + e4) continue;
                const int e = 4 * v_half + ((e4 + v_g) & 3); // rotate the channel order per lane: spreads LDS banks
                // byte e of each of the four tokens; the byte index is a run-time value, so the
                // v_perm selector is built instead of templated
                const uint32_t sel = 0x0c000c00u | (uint32_t)(e & 3) | ((uint32_t)(4 + (e & 3)) << 16);
                const bool upper = e >= 4;
                const uint32_t w0 = upper ? v_raw[0][1] : v_raw[0][0], w1 = upper ? v_raw[1][1] : v_raw[1][0];
                const uint32_t w2 = upper ? v_raw[2][1] : v_raw[2][0], w3 = upper ? v_raw[3][1] : v_raw[3][0];
                const half2_t lo = pk_sub_1152(__builtin_amdgcn_perm(w1, w0, sel) ^ 0x64806480u);
                const half2_t hi = pk_sub_1152(__builtin_amdgcn_perm(w3, w2, sel) ^ 0x64806480u);
                const half2_t h01 = lo * s01, h23 = hi * s23;
                u32x2 out, outl;
                out[0] = bitcast<uint32_t>(h01);
                out[1] = bitcast<uint32_t>(h23);
                outl[0] = bitcast<uint32_t>(__builtin_elementwise_fma(lo, s01, -h01));
                outl[1] = bitcast<uint32_t>(__builtin_elementwise_fma(hi, s23, -h23));
                *(u32x2*)&sV[(8 * v_g + e) * V_STRIDE + posv] = out;
                *(u32x2*)&sVlo[(8 * v_g + e) * V_STRIDE + posv] = outl;
            }
        }
    };

    auto store_tile = [&](int buf) {
#pragma unroll
        for (int k = 0; k < N_SLICES; ++k) store_slice(buf, k);
    };

    // Prologue: tile 0 dequantised into buffer 0, raw bytes of tile 1 in registers.
    int64_t row_next = 0;
    if (n_tiles > 0) {
        load_tile(0, tile_row(0));
        store_tile(0);
        if (n_tiles > 1) load_tile(1, tile_row(1));
        row_next = tile_row(2);
        __syncthreads();
    }
    // tokens this wave's columns attend to: beyond them (a tile past its columns' limits, or a wave whose columns lie
    // beyond the query rows: short chunks leave most waves without any) the wave only helps to stage the tiles
    int wave_lim = lim;
#pragma unroll
    for (int sh = 32; sh >= 1; sh >>= 1) {
        const int o = __shfl_xor(wave_lim, sh);
        wave_lim = o > wave_lim ? o : wave_lim;
    }
    wave_lim = __builtin_amdgcn_readfirstlane(wave_lim);
    for (int tile = 0; tile < n_tiles; ++tile) {
        const bool work = tile * kBN < wave_lim;
        const half_t* const sK = smem + (tile & 1) * TILE_HALVES;
        const half_t* const sKlo = sK + kBN * K_STRIDE;
        const half_t* const sV = KV16 ? sKlo : sKlo + kBN * K_STRIDE;
        const half_t* const sVlo = sV + D * V_STRIDE;

        // ---- S^T = K Q^T : two 32-token blocks.  The A fragments come from LDS in batches of QB k-steps, the
        // next batch requested before the current one is multiplied, so that an MFMA never waits for the
        // read issued just before it ----
        f32x16 s_acc[2];
#pragma unroll
        for (int mb = 0; mb < 2; ++mb)
#pragma unroll
            for (int i = 0; i < 16; ++i) s_acc[mb][i] = 0.f;
        if (work) {
            constexpr int QB = 4;
            constexpr int PER_MB = KSTEPS / QB;
            constexpr int NBATCH = 2 * PER_MB;
            f16x8 fh[2][QB], fl[2][QB];
            auto read_batch = [&](int bi, f16x8* ph, f16x8* pl) {
                const int mb = bi / PER_MB, s0 = (bi % PER_MB) * QB;
#pragma unroll
                for (int j = 0; j < QB; ++j) {
                    ph[j] = *(const f16x8*)&sK[(32 * mb + l32) * K_STRIDE + 16 * (s0 + j) + 8 * hh];
                    if (!KV16) pl[j] = *(const f16x8*)&sKlo[(32 * mb + l32) * K_STRIDE + 16 * (s0 + j) + 8 * hh];
                }
            };
            read_batch(0, fh[0], fl[0]);
#pragma unroll
            for (int bi = 0; bi < NBATCH; ++bi) {
                if (bi + 1 < NBATCH) read_batch(bi + 1, fh[(bi + 1) & 1], fl[(bi + 1) & 1]);
                __builtin_amdgcn_sched_barrier(0); // keep the requests ahead of the products (the scheduler would sink them)
                const int mb = bi / PER_MB, s0 = (bi % PER_MB) * QB;
#pragma unroll
                for (int j = 0; j < QB; ++j) {
                    if (!KV16) s_acc[mb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fl[bi & 1][j], qf[s0 + j], s_acc[mb], 0, 0, 0);
                    s_acc[mb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fh[bi & 1][j], qf[s0 + j], s_acc[mb], 0, 0, 0);
                }
                // between the batches: slices of tile + 1 into the other buffer (every wave is past its reads of
                // that buffer since the barrier that ended the previous iteration; after the last tile the slices
                // rewrite stale bytes into the idle buffer, which keeps this code free of branches)
#pragma unroll
                for (int k = 0; k < N_SLICES; ++k)
                    if (bi == k * NBATCH / N_SLICES) store_slice((tile & 1) ^ 1, k);
            }
        } else {
#pragma unroll
            for (int k = 0; k < N_SLICES; ++k) store_slice((tile & 1) ^ 1, k);
        }

        // ---- then the raw bytes of tile + 2 ----
        if (tile + 2 < n_tiles) {
            load_tile(tile + 2, row_next);
            row_next = tile_row(tile + 3);
        }

        if (work) {
            // ---- online softmax per column (element i <-> token 32 mb + 8 (i/4) + 4 hh + i%4) ----
            const int t_base = tile * kBN;
            // only the tiles that reach beyond a column's limit need the per-element test (wave-uniform branch)
            const bool need_mask = __builtin_amdgcn_ballot_w64(t_base + kBN > lim) != 0;
            float mx = kNegBig;
            if (EXTRA) {
                // additive terms per element (log2 units): mask value and alibi distance of (query row, token)
#pragma unroll
                for (int mb = 0; mb < 2; ++mb)
#pragma unroll
                    for (int i = 0; i < 16; ++i) {
                        const int t = t_base + 32 * mb + 8 * (i >> 2) + 4 * hh + (i & 3);
                        float v = -INFINITY;
                        if (t < lim) {
                            float add = 0.f;
                            if (mask_row) add = (float)mask_row[t];
                            if (a.alibi_slopes) add += a.is_causal ? slope * (float)t : -slope * fabsf((float)(pos_c + kvlen - qlen - t));
                            v = __builtin_fmaf(s_acc[mb][i], sm_scale, add * kLog2e);
                        }
                        s_acc[mb][i] = v;
                        mx = fmaxf(mx, v);
                    }
            } else {
                // maximum of the raw dot products; the (positive) logit scale is applied to it afterwards
                if (need_mask) {
#pragma unroll
                    for (int mb = 0; mb < 2; ++mb)
#pragma unroll
                        for (int i = 0; i < 16; ++i) {
                            const int t = t_base + 32 * mb + 8 * (i >> 2) + 4 * hh + (i & 3);
                            if (t >= lim) s_acc[mb][i] = -INFINITY;
                        }
                }
#pragma unroll
                for (int mb = 0; mb < 2; ++mb)
#pragma unroll
                    for (int i = 0; i < 16; ++i) mx = fmaxf(mx, s_acc[mb][i]);
                mx *= sm_scale;
            }
            mx = fmaxf(mx, __shfl_xor(mx, 32));
            const float m_new = fmaxf(m_run, mx);
            // the running max moves rarely once a few tiles have been seen: rescale only then (wave-uniform)
            if (__builtin_amdgcn_ballot_w64(m_new > m_run) != 0) {
                const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
                l_run *= alpha;
#pragma unroll
                for (int cb = 0; cb < CB; ++cb)
#pragma unroll
                    for (int i = 0; i < 16; ++i) o_acc[cb][i] *= alpha;
                m_run = m_new;
            }
            const float bias = kPShift - m_run;
            // p = hi + lo in halves: hi = p rounded toward zero (two at a time), lo = the exact remainder
            f16x8 pf[2][2], pfl[2][2];
            float lsum = 0.f;
#pragma unroll
            for (int mb = 0; mb < 2; ++mb)
#pragma unroll
                for (int i = 0; i < 16; i += 2) {
                    const float p0 = __builtin_amdgcn_exp2f(EXTRA ? s_acc[mb][i] + bias : __builtin_fmaf(s_acc[mb][i], sm_scale, bias));
                    const float p1 = __builtin_amdgcn_exp2f(EXTRA ? s_acc[mb][i + 1] + bias : __builtin_fmaf(s_acc[mb][i + 1], sm_scale, bias));
                    lsum += p0 + p1;
                    const half2_t ph = bitcast<half2_t>(__builtin_amdgcn_cvt_pkrtz(p0, p1));
                    const half2_t pl = bitcast<half2_t>(__builtin_amdgcn_cvt_pkrtz(sub_half_lo(p0, ph), sub_half_hi(p1, ph)));
                    pf[mb][i >> 3][i & 7] = ph.x;
                    pf[mb][i >> 3][(i & 7) + 1] = ph.y;
                    pfl[mb][i >> 3][i & 7] = pl.x;
                    pfl[mb][i >> 3][(i & 7) + 1] = pl.y;
                }
            l_run += lsum;

            // ---- O^T += V^T P^T : fragment batches of one (32-token block, 16-token step) each, read one ahead ----
            {
                f16x8 vh[2][CB], vl[2][CB];
                auto read_batch = [&](int bi, f16x8* ph, f16x8* pl) {
                    const int mb = bi >> 1, t = bi & 1;
#pragma unroll
                    for (int cb = 0; cb < CB; ++cb) {
                        ph[cb] = *(const f16x8*)&sV[(32 * cb + l32) * V_STRIDE + 32 * mb + 16 * t + 8 * hh];
                        if (!KV16) pl[cb] = *(const f16x8*)&sVlo[(32 * cb + l32) * V_STRIDE + 32 * mb + 16 * t + 8 * hh];
                    }
                };
                read_batch(0, vh[0], vl[0]);
#pragma unroll
                for (int bi = 0; bi < 4; ++bi) {
                    if (bi + 1 < 4) read_batch(bi + 1, vh[(bi + 1) & 1], vl[(bi + 1) & 1]);
                    __builtin_amdgcn_sched_barrier(0);
                    const int mb = bi >> 1, t = bi & 1;
#pragma unroll
                    for (int cb = 0; cb < CB; ++cb) {
                        if (!KV16) o_acc[cb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vl[bi & 1][cb], pf[mb][t], o_acc[cb], 0, 0, 0);
                        o_acc[cb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vh[bi & 1][cb], pfl[mb][t], o_acc[cb], 0, 0, 0);
                        o_acc[cb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vh[bi & 1][cb], pf[mb][t], o_acc[cb], 0, 0, 0);
                    }
                }
            }
        }
        __syncthreads(); // tile + 1 is complete in its buffer; this tile's buffer may be overwritten
    }

    // ---- normalise and store: element i of block cb <-> channel 32 cb + 8 (i/4) + 4 hh + i%4 ----
    const float l_tot = l_run + __shfl_xor(l_run, 32);
    const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
    if (col_on) {
        half_t* op = (half_t*)a.output + (q_row0 + pos) * a.output_stride_s + (int64_t)h * D;
#pragma unroll
        for (int cb = 0; cb < CB; ++cb)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                f16x4 w;
#pragma unroll
                for (int e = 0; e < 4; ++e) w[e] = (half_t)(o_acc[cb][4 * r + e] * inv);
                *(f16x4*)(op + 32 * cb + 8 * r + 4 * hh) = w;
            }
    }
}

template <int D, int SRC>
constexpr size_t prefill_lds_bytes()
{
    // int8 source: K hi/lo tiles + transposed V hi/lo tiles (above the 64 KB static limit for D = 128, hence
    // dynamic); fp16 source: one K tile and one transposed V tile; two buffers of each
    return 2 * (SRC == 2 ? 1 : 2) * (kBN * (D + 8) + D * (kBN + 8)) * sizeof(half_t);
}

template <int D, int SRC, bool EXTRA>
static std::atomic<int>& prefill_variant_ready()
{
    static std::atomic<int> ready{0};
    return ready;
}

template <int D, int SRC, bool EXTRA>
static int launch_prefill_variant(const PrefillLaunch& a, dim3 grid, hipStream_t stream)
{
    constexpr size_t lds_bytes = prefill_lds_bytes<D, SRC>();
    if (int rc = ensure_dynamic_lds((const void*)prefill_attention_kernel<D, SRC, EXTRA>, (int)lds_bytes, stream,
                                    prefill_variant_ready<D, SRC, EXTRA>()))
        return rc;
    hipLaunchKernelGGL((prefill_attention_kernel<D, SRC, EXTRA>), grid, dim3(kPrefillThreads), lds_bytes, stream, a);
    return kLaunchOk;
}

template <int D>
static int launch_prefill_d(const PrefillLaunch& a, hipStream_t stream)
{
    const int G = (int)(a.num_heads / a.num_kv_heads);
    const int ppw = kCols / G > 0 ? kCols / G : 1;
    // one workgroup per (query tile, kv head) that the batch can have at most; the kernel numbers the real ones first.
    // Every sequence has at most the tiles of max_seqlen; all together at most one per ppw rows plus a partial one each.
    int64_t items = a.prefill_batches * ((a.max_seqlen + ppw - 1) / ppw);
    if (a.query_rows > 0 && a.prefill_batches <= 64 * kPickSlots) {
        const int64_t by_rows = a.query_rows / ppw + a.prefill_batches;
        if (by_rows < items) items = by_rows;
    }
    const dim3 grid((unsigned)(items * a.num_kv_heads), 1, 1);
    const bool extra = a.attn_mask != nullptr || a.alibi_slopes != nullptr;
    const int src = a.current_key ? 2 : (a.cache_mode == 1 ? 0 : 1);
    if (extra) {
        if (src == 0) return launch_prefill_variant<D, 0, true>(a, grid, stream);
        if (src == 1) return launch_prefill_variant<D, 1, true>(a, grid, stream);
        return launch_prefill_variant<D, 2, true>(a, grid, stream);
    }
    if (src == 0) return launch_prefill_variant<D, 0, false>(a, grid, stream);
    if (src == 1) return launch_prefill_variant<D, 1, false>(a, grid, stream);
    return launch_prefill_variant<D, 2, false>(a, grid, stream);
}

int launch_prefill(const PrefillLaunch& a, hipStream_t stream)
{
    if (a.num_heads / a.num_kv_heads > kCols) return kLaunchNoKernel;
    switch (a.head_dim) {
        case 64: return launch_prefill_d<64>(a, stream);
        case 128: return launch_prefill_d<128>(a, stream);
        default: return kLaunchNoKernel;
    }
}

template <int D, int SRC, bool EXTRA>
static int init_prefill_variant()
{
    std::atomic<int>& ready = prefill_variant_ready<D, SRC, EXTRA>();
    if (ready.load() != 0) return kLaunchOk;
    if (hipFuncSetAttribute((const void*)prefill_attention_kernel<D, SRC, EXTRA>, hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)prefill_lds_bytes<D, SRC>()) != hipSuccess)
        return kLaunchNoKernel;
    ready.store(1);
    return kLaunchOk;
}
template <int D>
static int init_prefill_d()
{
    if (int rc = init_prefill_variant<D, 0, false>()) return rc;
    if (int rc = init_prefill_variant<D, 0, true>()) return rc;
    if (int rc = init_prefill_variant<D, 1, false>()) return rc;
    if (int rc = init_prefill_variant<D, 1, true>()) return rc;
    if (int rc = init_prefill_variant<D, 2, false>()) return rc;
    return init_prefill_variant<D, 2, true>();
}
int init_prefill_kernels()
{
    if (int rc = init_prefill_d<64>()) return rc;
    return init_prefill_d<128>();
}

} // namespace pmxhip
