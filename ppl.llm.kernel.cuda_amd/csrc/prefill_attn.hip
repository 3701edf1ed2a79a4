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
//     two MFMA stages.  V lies row-major ([token][channel], like K) in LDS and its
//     A fragments (rows = channels) are read with transposing 8-byte LDS loads
//     in the token order that layout asks for.
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

// LDS tile geometry.  K rows carry 16 bytes of padding: the 16-byte fragment reads of 32 rows then cover all banks.
// V rows are read with transposing 8-byte loads that take 64 bytes of each of four consecutive rows per
// half-wave: a row stride of 64 bytes modulo 256 puts those four segments on different banks.
template <int D>
struct PrefillTile {
    static constexpr int K_STRIDE = D + 8;
    static constexpr int V_STRIDE = ((D + 32) * 2) % 128 == 64 ? D + 32 : D + 64;
};
// first half of the epilogue's staging area: the start of the second tile buffer
template <int D, int SRC>
constexpr int kEpilogueBase()
{
    return (SRC == 2 ? 1 : 2) * kBN * (PrefillTile<D>::K_STRIDE + PrefillTile<D>::V_STRIDE);
}
static_assert((PrefillTile<128>::V_STRIDE * 2) % 256 == 64 && (PrefillTile<64>::V_STRIDE * 2) % 256 == 192 &&
                  (PrefillTile<96>::V_STRIDE * 2) % 256 == 64,
              "V row stride");

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
//
// Schedule of one 64-token tile in one wave (the two 32-token blocks b0, b1 of the tile are independent until the
// output accumulators).  Every phase pairs matrix work of one block with vector work of the other, in one
// instruction stream whose order is fixed by scheduling barriers:
//     phase 1   S^T(b0) products        with   dequantisation of the next tile into the other LDS buffer
//     phase 2   S^T(b1) products        with   softmax of b0 (and the global requests for the tile after next)
//     phase 3   O^T += V^T P^T of b0    with   softmax of b1
//     phase 4   O^T += V^T P^T of b1
// The running maximum is updated per block.  A maximum that moves rescales the accumulators (wave-uniform,
// rare after the first tiles): for b0 before its products start, for b1 after the products of b0 have been
// issued (the rescale then waits for them, being a reader of their accumulators).
//
// Measured on the mixed workload (16 sequences of 256-1024 query rows over up to 2048 prior tokens, 32 query / 8 kv
// heads of 128): the kernel takes 655 us; built without its products 442 us, without the LDS fragment reads 543 us,
// without dequantisation and global loads 531 us, without exp and the split of p 673 us, without the tile barrier
// 662 us, with none of these 131 us: the parts add up to the whole, so little of them runs concurrently.  The
// fragment reads alone take what the LDS port allows (512 KB per tile and CU at 256 bytes per clock).  A form with
// four waves of 64 columns (half the fragment reads per product, fragments requested two steps ahead, the whole
// register file per wave) took 1094 us: one wave per SIMD exposes every wait that a second wave covers.
template <int D, int SRC, bool EXTRA>
__global__ __launch_bounds__(kPrefillThreads, 2) void prefill_attention_kernel(const PrefillLaunch a)
{
    constexpr bool PAGED = SRC == 0;
    constexpr bool KV16 = SRC == 2;
    constexpr int KSTEPS = D / 16;          // MFMA k-steps over channels for S
    constexpr int CB = D / 32;              // 32-channel blocks of O^T
    constexpr int GPT = D / 8;              // quantisation groups per token row
    constexpr int K_STRIDE = PrefillTile<D>::K_STRIDE; // halves per K row in LDS
    constexpr int V_STRIDE = PrefillTile<D>::V_STRIDE; // halves per V row in LDS (row-major, like K)
    // Staging: thread t takes group t % GPT of the tokens t / GPT, t / GPT + K_TSTEP, ...  With 12 groups per row
    // (head_dim 96) the first 384 threads stage 32 tokens per pass and the last two waves stage nothing.
    constexpr int K_TSTEP = GPT == 12 ? 32 : kPrefillThreads / GPT; // tokens between a thread's units
    constexpr int STAGERS = K_TSTEP * GPT;                           // threads that stage (whole waves)
    constexpr int UNITS = kBN / K_TSTEP;                             // (token, group) units per staging thread, of K and of V each
    static_assert(STAGERS <= kPrefillThreads && STAGERS % 64 == 0 && UNITS * K_TSTEP == kBN, "staging units");

    // K is kept as an unevaluated sum hi + lo of two halves: hi = fp16(int8 * scale) and
    // lo = the rounding error of that product (exact, from one fused multiply-add), so that
    // q.k carries no fp16 rounding of the dequantised key.  With a single rounded copy a
    // 2^-12 relative error on |q_c k_c| ~ 1e3 (outlier channels) moves logits by ~1e-2.
    // V and the probabilities are split the same way (V^ = hi + lo from the same multiply-add
    // trick, p = hi + lo), and O accumulates hi*hi + lo*hi + hi*lo: at |v| ~ 40 a single fp16
    // rounding of either factor already costs ~1e-2 absolute where contributions cancel.
    extern __shared__ __attribute__((aligned(16))) char smem_raw[];
    // two tile buffers; a buffer holds K (hi, lo) and V (hi, lo), all row-major [token][channel]
    // (fp16 K/V need no low parts: the tiles are the values themselves)
    constexpr int K_HALVES = kBN * K_STRIDE, V_HALVES = kBN * V_STRIDE;
    constexpr int TILE_HALVES = (KV16 ? 1 : 2) * (K_HALVES + V_HALVES);
    half_t* const smem = (half_t*)smem_raw;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int hh = lane >> 5;   // half-wave
    const int l32 = lane & 31;

    // per-lane parts of the LDS addresses (halves)
    const int k_frag_off = l32 * K_STRIDE + 8 * hh; // + (32 mb) rows + 16 s: the A fragment of S^T
    // A fragment of O^T = rows (channels) of V^T, read from the row-major tile with transposing loads: in a group
    // of 16 lanes, lane i sends the address of 4 channels (4 (i % 4) ..) of token (i / 4) and receives channel i
    // of the group's 4 tokens.  The group (lane / 16) = (channel half g % 2, token half hh).
    const int v_frag_off = (4 * hh + ((lane & 15) >> 2)) * V_STRIDE + 16 * ((lane >> 4) & 1) + 4 * (lane & 3);

    const int G = (int)(a.num_heads / a.num_kv_heads);
    const int ppw = kCols / G > 0 ? kCols / G : 1; // query positions per workgroup
    const int kvh = blockIdx.x % (int)a.num_kv_heads;
    const int item_stride = gridDim.x / (int)a.num_kv_heads;

    const int8_t* __restrict__ cache = (const int8_t*)a.cache;
    const half_t* __restrict__ scale = (const half_t*)a.scale;
    const int64_t head_off = a.layer_idx * a.cache_stride_l + (int64_t)kvh * a.cache_stride_h;
    const int8_t* const cache_k = cache + head_off;
    const int8_t* const cache_v = cache_k + a.cache_stride_kv;
    const half_t* const scale_k = scale + (head_off >> 3);
    const half_t* const scale_v = scale_k + (a.cache_stride_kv >> 3);
    const const_i64_ptr cachestarts = as_constant(a.cachestarts);
    const float sm_scale = a.attn_scale * kLog2e;

    // this thread's (token, group) units of a tile: token u_t0 + u * K_TSTEP, group u_g, for K and for V alike
    const bool stager = tid < STAGERS; // wave-uniform
    const int u_g = tid % GPT;
    const int u_t0 = stager ? tid / GPT : 0;
    const uint32_t stride_s32 = (uint32_t)a.cache_stride_s; // the host checks that a tile's span fits 32 bits
    const uint32_t kstride16 = (uint32_t)a.key_stride_s, vstride16 = (uint32_t)a.value_stride_s;
    uint32_t u_off[UNITS];
#pragma unroll
    for (int u = 0; u < UNITS; ++u) u_off[u] = (uint32_t)(u_t0 + u * K_TSTEP) * stride_s32 + 8 * u_g;

    // The workgroups of the launch share the batch's query tiles: workgroup (item, kv head) takes the items
    // item, item + item_stride, ... in the order of falling cost, so that a launch that was sized from a hint that
    // understates the batch still covers every tile (it only takes longer).
    for (int item = blockIdx.x / (int)a.num_kv_heads;; item += item_stride) {
    int b_pick = 0, tile_pick = 0;
    if (!pick_query_tile(a, ppw, item, lane, b_pick, tile_pick)) return;
    const int b = __builtin_amdgcn_readfirstlane(b_pick);
    const int64_t q_row0 = a.seqstarts[b];
    const int qlen = (int)(a.seqstarts[b + 1] - q_row0);
    const int kvlen = (int)(a.kvstarts[b + 1] - a.kvstarts[b]);
    const int p0 = __builtin_amdgcn_readfirstlane(tile_pick) * ppw;
    if (p0 < 0 || p0 >= qlen) continue;

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
    // element (head, absolute query row, absolute kv column) of the additive mask; kvstarts holds absolute columns
    const half_t* mask_row = nullptr;
    float slope = 0.f;
    if (EXTRA) {
        if (a.attn_mask)
            mask_row = (const half_t*)a.attn_mask + (int64_t)h * a.mask_stride_h + (q_row0 + pos_c) * a.mask_stride_s + a.kvstarts[b];
        if (a.alibi_slopes) slope = a.alibi_slopes[h];
    }

    // ---- global -> register staging of one tile's raw bytes ----
    const int64_t table_base = PAGED ? (int64_t)b * a.cachestarts_stride_b : (int64_t)b;
    u32x2 k_raw[UNITS], v_raw[UNITS];
    half_t k_sc[UNITS], v_sc[UNITS];
    u32x4 k16[UNITS], v16[UNITS]; // fp16 source: 8 halves per unit

    // Addressing: a tile of 64 tokens starts at a multiple of 64, so it lies inside one page.  Its row
    // base is wave-uniform (scalar loads of the page table, read one tile ahead); the per-lane part
    // (token in tile, channel group) never changes and is computed once.
    auto tile_row = [&](int tile) -> int64_t {
        int t_base = tile * kBN;
        if (t_base > kvlen - 1) t_base = kvlen > 0 ? kvlen - 1 : 0;
        if (KV16) return q_row0 + t_base; // current_key row of kv token t = query row of the same position
        if (PAGED) return cachestarts[table_base + (t_base >> 7)] + (t_base & (kPage - 1));
        return cachestarts[table_base] + t_base;
    };
    auto load_tile = [&](int tile, int64_t row) {
        if (!stager) return;
        const int left = kvlen - 1 - tile * kBN; // offset of the sequence's last token inside this tile
        if (KV16) {
            const half_t* bk = (const half_t*)a.current_key + row * a.key_stride_s + (int64_t)kvh * D;
            const half_t* bv = (const half_t*)a.current_value + row * a.value_stride_s + (int64_t)kvh * D;
#pragma unroll
            for (int u = 0; u < UNITS; ++u) {
                int t = u_t0 + u * K_TSTEP;
                t = t < left ? t : (left > 0 ? left : 0);
                k16[u] = *(const u32x4*)(bk + (uint32_t)t * kstride16 + 8 * u_g);
                v16[u] = *(const u32x4*)(bv + (uint32_t)t * vstride16 + 8 * u_g);
            }
            return;
        }
        const int64_t boff = row * a.cache_stride_s;
        const int8_t* bk = cache_k + boff;
        const int8_t* bv = cache_v + boff;
        const half_t* sk = scale_k + (boff >> 3);
        const half_t* sv = scale_v + (boff >> 3);
        if (left >= kBN - 1) {
#pragma unroll
            for (int u = 0; u < UNITS; ++u) {
                k_raw[u] = *(const u32x2*)(bk + u_off[u]);
                k_sc[u] = sk[u_off[u] >> 3];
                v_raw[u] = *(const u32x2*)(bv + u_off[u]);
                v_sc[u] = sv[u_off[u] >> 3];
            }
        } else { // last tile of the sequence: tokens beyond it re-read its last token (masked later)
#pragma unroll
            for (int u = 0; u < UNITS; ++u) {
                const int t = u_t0 + u * K_TSTEP;
                const uint32_t off = (uint32_t)(t < left ? t : (left > 0 ? left : 0)) * stride_s32 + 8 * u_g;
                k_raw[u] = *(const u32x2*)(bk + off);
                k_sc[u] = sk[off >> 3];
                v_raw[u] = *(const u32x2*)(bv + off);
                v_sc[u] = sv[off >> 3];
            }
        }
    };
    // One slice of the dequantise-and-store of a tile: slices [0, UNITS) are this thread's K units, slices
    // UNITS + [0, UNITS) its V units.  Sliced so that the work can be spread between the MFMAs of phase 1.
    constexpr int N_SLICES = 2 * UNITS;
    auto store_slice = [&](int buf, int slice) {
        if (!stager) return;
        half_t* const sK = smem + buf * TILE_HALVES;
        half_t* const sKlo = sK + K_HALVES;
        half_t* const sV = KV16 ? sKlo : sKlo + K_HALVES;
        half_t* const sVlo = sV + V_HALVES;
        const bool is_v = slice >= UNITS;
        const int u = is_v ? slice - UNITS : slice;
        const int t = u_t0 + u * K_TSTEP;
        half_t* const dst = is_v ? &sV[t * V_STRIDE + 8 * u_g] : &sK[t * K_STRIDE + 8 * u_g];
        if (KV16) {
            *(u32x4*)dst = is_v ? v16[u] : k16[u];
            return;
        }
        half_t* const dst_lo = is_v ? &sVlo[t * V_STRIDE + 8 * u_g] : &sKlo[t * K_STRIDE + 8 * u_g];
        const u32x2 raw = is_v ? v_raw[u] : k_raw[u];
        const half_t scl = is_v ? v_sc[u] : k_sc[u];
        const half2_t sc = {scl, scl};
        const uint32_t f0 = raw[0] ^ kFlipSigns, f1 = raw[1] ^ kFlipSigns;
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
        *(u32x4*)dst = w;
        *(u32x4*)dst_lo = wl;
    };

    // Prologue: tile 0 dequantised into buffer 0, raw bytes of tile 1 in registers.
    int64_t row_next = 0;
    if (n_tiles > 0) {
        load_tile(0, tile_row(0));
#pragma unroll
        for (int k = 0; k < N_SLICES; ++k) store_slice(0, k);
        if (n_tiles > 1) load_tile(1, tile_row(1));
        row_next = tile_row(2);
        __syncthreads();
    }
    // tokens this wave's columns attend to: beyond the largest limit (a tile past its columns' limits, or a wave
    // whose columns lie beyond the query rows: short chunks leave most waves without any) the wave only helps to
    // stage the tiles; up to the smallest limit of its live columns no element needs the limit test
    int wave_lim = lim, wave_lim_min = col_on ? lim : 0x7fffffff;
#pragma unroll
    for (int sh = 32; sh >= 1; sh >>= 1) {
        const int o = __shfl_xor(wave_lim, sh), o2 = __shfl_xor(wave_lim_min, sh);
        wave_lim = o > wave_lim ? o : wave_lim;
        wave_lim_min = o2 < wave_lim_min ? o2 : wave_lim_min;
    }
    wave_lim = __builtin_amdgcn_readfirstlane(wave_lim);
    wave_lim_min = __builtin_amdgcn_readfirstlane(wave_lim_min);

    // ---- one tile, for a wave that has columns in it.  limit: some element may lie beyond its column's limit ----
    auto tile_body = [&](int tile, const bool limit) {
        const int buf = tile & 1;
        const half_t* const sK = smem + buf * TILE_HALVES;
        const half_t* const sKlo = sK + K_HALVES;
        const half_t* const sV = KV16 ? sKlo : sKlo + K_HALVES;
        const half_t* const sVlo = sV + V_HALVES;
        const int t_base = tile * kBN;

        // K fragments of block mb, k-steps s0, s0 + 1 (hi and lo)
        constexpr int QB = 1;                  // k-steps per batch
        constexpr int NQB = KSTEPS / QB;       // batches per block
        auto read_k = [&](int mb, int qb, f16x8* fh, f16x8* fl) {
#pragma unroll
            for (int j = 0; j < QB; ++j) {
                fh[j] = *(const f16x8*)&sK[k_frag_off + 32 * mb * K_STRIDE + 16 * (qb * QB + j)];
                if (!KV16) fl[j] = *(const f16x8*)&sKlo[k_frag_off + 32 * mb * K_STRIDE + 16 * (qb * QB + j)];
            }
        };
        auto mul_k = [&](f32x16& acc, int qb, const f16x8* fh, const f16x8* fl) {
#pragma unroll
            for (int j = 0; j < QB; ++j) {
                if (!KV16) acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(fl[j], qf[qb * QB + j], acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(fh[j], qf[qb * QB + j], acc, 0, 0, 0);
            }
        };
        // V^T fragments of block mb, 16-token step t, channel blocks cb0, cb0 + 1: element j of a fragment is token
        // 32 mb + 16 t + 8 (j / 4) + 4 hh + j % 4, the token of element 8 t + j of the lane's S^T accumulator
        constexpr int VB = 1;                  // channel blocks per batch
        constexpr int NVB = 2 * CB / VB;       // batches per block: (t, pair of channel blocks)
        auto read_vt = [&](const half_t* base, int mb, int t, int cb) -> f16x8 {
            typedef short s16x4 __attribute__((ext_vector_type(4)));
            typedef __attribute__((address_space(3))) s16x4* lds_s16x4_ptr;
            const half_t* p = base + v_frag_off + (32 * mb + 16 * t) * V_STRIDE + 32 * cb;
            const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(p));
            const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(p + 8 * V_STRIDE));
            return bitcast<f16x8>(__builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
        };
        auto read_v = [&](int mb, int vb, f16x8* fh, f16x8* fl) {
            const int t = vb / (CB / VB), cb0 = (vb % (CB / VB)) * VB;
#pragma unroll
            for (int j = 0; j < VB; ++j) {
                fh[j] = read_vt(sV, mb, t, cb0 + j);
                if (!KV16) fl[j] = read_vt(sVlo, mb, t, cb0 + j);
            }
        };
        auto mul_v = [&](int vb, const f16x8* fh, const f16x8* fl, const f16x8* ph, const f16x8* pl) {
            const int t = vb / (CB / VB), cb0 = (vb % (CB / VB)) * VB;
#pragma unroll
            for (int j = 0; j < VB; ++j) {
                if (!KV16) o_acc[cb0 + j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fl[j], ph[t], o_acc[cb0 + j], 0, 0, 0);
                o_acc[cb0 + j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fh[j], pl[t], o_acc[cb0 + j], 0, 0, 0);
                o_acc[cb0 + j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fh[j], ph[t], o_acc[cb0 + j], 0, 0, 0);
            }
        };

        // ---- softmax of one block, in three parts so that products can be issued between them ----
        // part A: the block's logits in log2 units where extra terms or limits apply, and the new running maximum
        auto softmax_max = [&](f32x16& sacc, int mb) -> float {
            float mx = kNegBig;
            if (EXTRA) {
                // element i is token t0 + o_i, o_i = 8 (i / 4) + i % 4 a constant of the unrolled loop.  The alibi term
                // is slope2 * (t0 + o_i) (causal) or -slope2 * |d0 - o_i| with d0 the distance of t0 from the column's
                // own position: one multiply-add per element on a per-block base.  The limit test runs only on the
                // tiles that reach a column's limit, as in the plain form; mask values are read below the limit only
                // (the tile may reach beyond the mask's row).
                const int t0 = t_base + 32 * mb + 4 * hh;
                const float slope2 = slope * kLog2e;
                const bool has_alibi = a.alibi_slopes != nullptr, causal = a.is_causal != 0;
                const float base = causal ? slope2 * (float)t0 : (float)(pos_c + kvlen - qlen - t0);
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const int o = 8 * (i >> 2) + (i & 3);
                    float add = 0.f;
                    if (has_alibi) add = causal ? __builtin_fmaf(slope2, (float)o, base) : -slope2 * fabsf(base - (float)o);
                    if (mask_row && t0 + o < lim) add = __builtin_fmaf((float)mask_row[t0 + o], kLog2e, add);
                    float v = __builtin_fmaf(sacc[i], sm_scale, add);
                    if ((limit || mask_row) && t0 + o >= lim) v = -INFINITY;
                    sacc[i] = v;
                    mx = fmaxf(mx, v);
                }
            } else {
                if (limit) { // wave-uniform: only the tiles that reach beyond a column's limit
#pragma unroll
                    for (int i = 0; i < 16; ++i) {
                        const int t = t_base + 32 * mb + 8 * (i >> 2) + 4 * hh + (i & 3);
                        if (t >= lim) sacc[i] = -INFINITY;
                    }
                }
                // maximum of the raw dot products; the (positive) logit scale is applied to it afterwards
#pragma unroll
                for (int i = 0; i < 16; i += 2) mx = max3(mx, sacc[i], sacc[i + 1]);
                mx *= sm_scale;
            }
            {
                // the other half-wave's maximum through the vector unit's lane swap: a data-share permute would have
                // to wait for every fragment read already queued behind it
                const u32x2 both = __builtin_amdgcn_permlane32_swap(bitcast<uint32_t>(mx), bitcast<uint32_t>(mx), false, false);
                mx = fmaxf(bitcast<float>(both[0]), bitcast<float>(both[1]));
            }
            return fmaxf(m_run, mx);
        };
        // part B: p = 2^(logit - max) as hi + lo halves (hi = p rounded to nearest, two at a time; lo = the exact
        // remainder), elements [i0, i1) of the block.  The row sum is taken over the hi halves, one dot-product
        // instruction per pair instead of two additions: rounded to nearest, their errors are at most 2^-12 of each
        // term and of either sign, so the sum of a row's hundreds of terms differs from the sum of p by ~1e-5 of itself
        // (a factor on the whole output row, against a relative tolerance of 1e-2).
        auto softmax_exp = [&](const f32x16& sacc, float bias, int i0, int i1, f16x8* ph, f16x8* pl, float& lsum) {
#pragma unroll
            for (int i = 0; i < 16; i += 2) {
                if (i < i0 || i >= i1) continue;
                const float p0 = __builtin_amdgcn_exp2f(EXTRA ? sacc[i] + bias : __builtin_fmaf(sacc[i], sm_scale, bias));
                const float p1 = __builtin_amdgcn_exp2f(EXTRA ? sacc[i + 1] + bias : __builtin_fmaf(sacc[i + 1], sm_scale, bias));
                typedef float float2_t __attribute__((ext_vector_type(2)));
                const half2_t h2 = __builtin_convertvector(float2_t{p0, p1}, half2_t);
                lsum = __builtin_amdgcn_fdot2(h2, half2_t{(half_t)1.f, (half_t)1.f}, lsum, false);
                const half2_t l2 = bitcast<half2_t>(__builtin_amdgcn_cvt_pkrtz(sub_half_lo(p0, h2), sub_half_hi(p1, h2)));
                ph[i >> 3][i & 7] = h2.x;
                ph[i >> 3][(i & 7) + 1] = h2.y;
                pl[i >> 3][i & 7] = l2.x;
                pl[i >> 3][(i & 7) + 1] = l2.y;
            }
        };
        auto rescale = [&](float m_new) {
            const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
            l_run *= alpha;
#pragma unroll
            for (int cb = 0; cb < CB; ++cb)
#pragma unroll
                for (int i = 0; i < 16; ++i) o_acc[cb][i] *= alpha;
            m_run = m_new;
        };
#define PMX_FENCE() __builtin_amdgcn_sched_barrier(0)

        f32x16 s0, s1;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            s0[i] = 0.f;
            s1[i] = 0.f;
        }
        f16x8 fh[2][QB > VB ? QB : VB], fl[2][QB > VB ? QB : VB];
        f16x8 p0h[2], p0l[2], p1h[2], p1l[2];

        // ---- phase 1: S^T(b0) with the dequantisation of tile + 1 into the other buffer (every wave is past its
        // reads of that buffer since the barrier that ended the previous iteration; after the last tile the slices
        // rewrite stale bytes into the idle buffer, which keeps this code free of branches) ----
        read_k(0, 0, fh[0], fl[0]);
#pragma unroll
        for (int qb = 0; qb < NQB; ++qb) {
            if (qb + 1 < NQB) read_k(0, qb + 1, fh[(qb + 1) & 1], fl[(qb + 1) & 1]);
            else read_k(1, 0, fh[(qb + 1) & 1], fl[(qb + 1) & 1]);
            PMX_FENCE();
            mul_k(s0, qb, fh[qb & 1], fl[qb & 1]);
            PMX_FENCE();
#pragma unroll
            for (int k = 0; k < N_SLICES; ++k)
                if (qb == k * NQB / N_SLICES) store_slice(buf ^ 1, k);
            PMX_FENCE();
        }

        // ---- phase 2: S^T(b1) with the softmax of b0 ----
        float lsum = 0.f;
        float m_new = 0.f, bias = 0.f;
#pragma unroll
        for (int qb = 0; qb < NQB; ++qb) {
            if (qb + 1 < NQB) read_k(1, qb + 1, fh[(NQB + qb + 1) & 1], fl[(NQB + qb + 1) & 1]);
            PMX_FENCE();
            mul_k(s1, qb, fh[(NQB + qb) & 1], fl[(NQB + qb) & 1]);
            PMX_FENCE();
            if (qb == 0) {
                // the raw bytes of tile + 2: their registers were freed by phase 1, and the requests have the rest of
                // this tile and phase 1 of the next to complete
                if (tile + 2 < n_tiles) {
                    load_tile(tile + 2, row_next);
                    row_next = tile_row(tile + 3);
                }
                m_new = softmax_max(s0, 0);
                // the running max moves rarely once a few tiles have been seen: rescale only then (wave-uniform)
                if (__builtin_amdgcn_ballot_w64(m_new > m_run) != 0) rescale(m_new);
                bias = kPShift - m_run;
            }
            if (NQB == 1) softmax_exp(s0, bias, 0, 16, p0h, p0l, lsum);
            else if (qb >= 1 || NQB == 2) {
                // the 16 elements over the remaining batches
                const int parts = NQB == 2 ? 2 : NQB - 1, part = NQB == 2 ? qb : qb - 1;
                softmax_exp(s0, bias, 16 * part / parts & ~1, 16 * (part + 1) / parts & ~1, p0h, p0l, lsum);
            }
            PMX_FENCE();
        }
        l_run += lsum;

        // ---- phase 3: O^T += V^T P^T of b0 with the softmax of b1 ----
        lsum = 0.f;
        float m_b1 = 0.f;
        read_v(0, 0, fh[0], fl[0]);
#pragma unroll
        for (int vb = 0; vb < NVB; ++vb) {
            if (vb + 1 < NVB) read_v(0, vb + 1, fh[(vb + 1) & 1], fl[(vb + 1) & 1]);
            else read_v(1, 0, fh[(vb + 1) & 1], fl[(vb + 1) & 1]);
            PMX_FENCE();
            mul_v(vb, fh[vb & 1], fl[vb & 1], p0h, p0l);
            PMX_FENCE();
            if (vb == 0) {
                m_b1 = softmax_max(s1, 1);
                bias = kPShift - m_b1; // b1's probabilities are taken against the maximum that includes b1
            }
            softmax_exp(s1, bias, 16 * vb / NVB & ~1, 16 * (vb + 1) / NVB & ~1, p1h, p1l, lsum);
            PMX_FENCE();
        }
        // b1 raised the maximum: what has been accumulated so far, the products of b0 included, is rescaled
        if (__builtin_amdgcn_ballot_w64(m_b1 > m_run) != 0) rescale(m_b1);
        l_run += lsum;

        // ---- phase 4: O^T += V^T P^T of b1; the raw bytes of tile + 2 are requested after the first batch ----
#pragma unroll
        for (int vb = 0; vb < NVB; ++vb) {
            if (vb + 1 < NVB) read_v(1, vb + 1, fh[(NVB + vb + 1) & 1], fl[(NVB + vb + 1) & 1]);
            PMX_FENCE();
            mul_v(vb, fh[(NVB + vb) & 1], fl[(NVB + vb) & 1], p1h, p1l);
            PMX_FENCE();
            PMX_FENCE();
        }
#undef PMX_FENCE
    };

    for (int tile = 0; tile < n_tiles; ++tile) {
        if (tile * kBN < wave_lim) {
            tile_body(tile, (tile + 1) * kBN > wave_lim_min);
        } else {
#pragma unroll
            for (int k = 0; k < N_SLICES; ++k) store_slice((tile & 1) ^ 1, k);
            if (tile + 2 < n_tiles) {
                load_tile(tile + 2, row_next);
                row_next = tile_row(tile + 3);
            }
        }
        __syncthreads(); // tile + 1 is complete in its buffer; this tile's buffer may be overwritten
    }

    // ---- normalise and store: element i of block cb <-> channel 32 cb + 8 (i/4) + 4 hh + i%4 ----
    // A lane holds 8-byte pieces of one output row; stored as they lie, every store instruction would touch 32 rows
    // with 16 bytes each, and the partly written lines would wait in the caches to be completed.  The wave turns its
    // 32 rows round in LDS instead (its own region of the second tile buffer: every wave is past the tile loop's last
    // barrier, and the next item writes that buffer only after its prologue's barrier, which this wave joins after this)
    // and writes whole rows, 16 bytes per lane, with the non-temporal hint: the rows are not read again by this
    // kernel, and lines left dirty in the memory-side cache are written back during whatever runs next (a decode launch
    // after 89 MB of such rows took 12 us longer).
    const float l_tot = l_run + __shfl_xor(l_run, 32);
    const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
    {
        constexpr int EP_STRIDE = D + 8;                  // halves per staged row (rows stay 16-byte aligned)
        constexpr int EP_WAVE = 32 * EP_STRIDE + 32 * 4;  // 32 rows, then their 64-bit output offsets
        half_t* const ep = smem + kEpilogueBase<D, SRC>() + wave * EP_WAVE;
        int64_t* const ep_off = (int64_t*)(ep + 32 * EP_STRIDE);
#pragma unroll
        for (int cb = 0; cb < CB; ++cb)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                f16x4 w;
#pragma unroll
                for (int e = 0; e < 4; ++e) w[e] = (half_t)(o_acc[cb][4 * r + e] * inv);
                *(f16x4*)(ep + l32 * EP_STRIDE + 32 * cb + 8 * r + 4 * hh) = w;
            }
        if (hh == 0) ep_off[l32] = col_on ? (q_row0 + pos) * a.output_stride_s + (int64_t)h * D : (int64_t)-1;
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        // 16-byte stores need rows that start on 16-byte addresses (wave-uniform: a property of the launch)
        const bool wide_rows = ((uintptr_t)a.output & 15u) == 0 && (a.output_stride_s & 7) == 0;
        constexpr int CH = D / 8;            // 16-byte pieces per row
        constexpr int RPI = 64 / CH;         // rows per store instruction
        const int piece = lane % CH, row_in = lane / CH;
#pragma unroll
        for (int r0 = 0; r0 < 32; r0 += RPI) {
            const int row = r0 + row_in;
            if (row_in < RPI && row < 32) {
                const int64_t off = ep_off[row];
                const u32x4 w = *(const u32x4*)(ep + row * EP_STRIDE + 8 * piece);
                if (off >= 0) {
                    half_t* const dst = (half_t*)a.output + off + 8 * piece;
                    if (wide_rows) {
                        __builtin_nontemporal_store(w, (u32x4*)dst);
                    } else { // output rows aligned to 8 bytes only
                        *(u32x2*)dst = u32x2{w[0], w[1]};
                        *(u32x2*)(dst + 4) = u32x2{w[2], w[3]};
                    }
                }
            }
        }
    }
    } // items
}

// ---- the 16-column form: head_dim 256, whose accumulators and query fragments the kernel above cannot hold ----
// (128 accumulator and 64 query registers per lane with 32 columns per wave).  Here a wave has 16 columns and the products run on
// v_mfma_f32_16x16x32_f16: S^T tiles of 16 tokens x 16 columns (4 registers), O^T tiles of 16 channels x 16 columns.
// Same decomposition otherwise (one workgroup = one kv head x a tile of query positions x all query heads of the
// group: 128 columns; K/V tiles dequantised once per workgroup into one of two LDS buffers, one barrier per tile;
// hi + lo pairs for K^, V^ and p), in a plain order: stage the next tile, then S^T, softmax, O^T of this one.
// A lane (column c = lane % 16, quarter kq = lane / 16) holds of each S^T tile the tokens 4 kq .. 4 kq + 3; a tile of
// 32 tokens is two S^T tiles, and its 8 values per lane are the lane's share of the k dimension of the O^T step
// (slot e of quarter kq = token 16 (e / 4) + 4 kq + e % 4), which is the order the transposing V reads deliver.
namespace {
constexpr int kBN16 = 32;    // kv tokens per tile
constexpr int kCols16 = 128; // (position, head) columns per workgroup, 16 per wave
template <int D>
struct PrefillTile16 {
    static constexpr int K_STRIDE = D + 8;
    static constexpr int V_STRIDE = ((D + 32) * 2) % 128 == 64 ? D + 32 : D + 64; // an odd multiple of 64 bytes
};
static_assert((PrefillTile16<256>::V_STRIDE * 2) % 128 == 64, "V row stride");
} // namespace

template <int D, int SRC, bool EXTRA>
__global__ __launch_bounds__(kPrefillThreads, D <= 128 ? 4 : 2) void prefill_attention16_kernel(const PrefillLaunch a)
{
    constexpr bool PAGED = SRC == 0;
    constexpr bool KV16 = SRC == 2;
    constexpr int KSTEPS = D / 32;          // MFMA k-steps over channels for S
    constexpr int CT = D / 16;              // 16-channel tiles of O^T
    constexpr int GPT = D / 8;              // quantisation groups per token row
    constexpr int K_STRIDE = PrefillTile16<D>::K_STRIDE;
    constexpr int V_STRIDE = PrefillTile16<D>::V_STRIDE;
    constexpr int TILE_UNITS = kBN16 * GPT; // (token, group) units of a tile, of K and of V each
    constexpr int UNITS = (TILE_UNITS + kPrefillThreads - 1) / kPrefillThreads;
    constexpr int K_HALVES = kBN16 * K_STRIDE, V_HALVES = kBN16 * V_STRIDE;
    constexpr int TILE_HALVES = (KV16 ? 1 : 2) * (K_HALVES + V_HALVES);

    extern __shared__ __attribute__((aligned(16))) char smem_raw[];
    half_t* const smem = (half_t*)smem_raw;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int r16 = lane & 15;
    const int kq = lane >> 4;
    const int k_frag_off = r16 * K_STRIDE + 8 * kq;                            // + 16 mb rows + 32 s
    const int v_frag_off = (4 * kq + (r16 >> 2)) * V_STRIDE + 4 * (lane & 3);  // + 16 rows for slots 4..7, + 16 ct

    const int G = (int)(a.num_heads / a.num_kv_heads);
    const int ppw = kCols16 / G > 0 ? kCols16 / G : 1;
    const int kvh = blockIdx.x % (int)a.num_kv_heads;
    const int item_stride = gridDim.x / (int)a.num_kv_heads;

    const int8_t* __restrict__ cache = (const int8_t*)a.cache;
    const half_t* __restrict__ scale = (const half_t*)a.scale;
    const int64_t head_off = a.layer_idx * a.cache_stride_l + (int64_t)kvh * a.cache_stride_h;
    const int8_t* const cache_k = cache + head_off;
    const int8_t* const cache_v = cache_k + a.cache_stride_kv;
    const half_t* const scale_k = scale + (head_off >> 3);
    const half_t* const scale_v = scale_k + (a.cache_stride_kv >> 3);
    const const_i64_ptr cachestarts = as_constant(a.cachestarts);
    const float sm_scale = a.attn_scale * kLog2e;

    // this thread's units of a tile: unit tid + 512 u = (token, group)
    const uint32_t stride_s32 = (uint32_t)a.cache_stride_s; // the host checks that a tile's span fits 32 bits
    const uint32_t kstride16 = (uint32_t)a.key_stride_s, vstride16 = (uint32_t)a.value_stride_s;
    int u_t[UNITS], u_g[UNITS];
    bool u_on[UNITS];
#pragma unroll
    for (int u = 0; u < UNITS; ++u) {
        const int idx = tid + u * kPrefillThreads;
        u_on[u] = idx < TILE_UNITS;
        u_t[u] = u_on[u] ? idx / GPT : 0;
        u_g[u] = u_on[u] ? idx % GPT : 0;
    }

    for (int item = blockIdx.x / (int)a.num_kv_heads;; item += item_stride) {
    int b_pick = 0, tile_pick = 0;
    if (!pick_query_tile(a, ppw, item, lane, b_pick, tile_pick)) return;
    const int b = __builtin_amdgcn_readfirstlane(b_pick);
    const int64_t q_row0 = a.seqstarts[b];
    const int qlen = (int)(a.seqstarts[b + 1] - q_row0);
    const int kvlen = (int)(a.kvstarts[b + 1] - a.kvstarts[b]);
    const int p0 = __builtin_amdgcn_readfirstlane(tile_pick) * ppw;
    if (p0 < 0 || p0 >= qlen) continue;

    // ---- this lane's column ----
    const int col = wave * 16 + r16;
    const int pos = p0 + col / G;
    const int g = col % G;
    const bool col_on = (col < ppw * G) && (pos < qlen);
    const int pos_c = pos < qlen ? pos : qlen - 1;
    const int h = kvh * G + (col < ppw * G ? g : 0);
    int lim = kvlen; // this column attends tokens [0, lim)
    if (a.is_causal) {
        lim = pos_c + 1 + kvlen - qlen;
        lim = lim < 0 ? 0 : (lim > kvlen ? kvlen : lim);
    }
    if (!col_on) lim = 0;
    int last_pos = p0 + ppw - 1;
    if (last_pos > qlen - 1) last_pos = qlen - 1;
    int wg_lim = kvlen;
    if (a.is_causal) {
        wg_lim = last_pos + 1 + kvlen - qlen;
        wg_lim = wg_lim < 0 ? 0 : (wg_lim > kvlen ? kvlen : wg_lim);
    }
    const int n_tiles = (wg_lim + kBN16 - 1) / kBN16;
    int wave_lim = lim;
#pragma unroll
    for (int sh = 32; sh >= 1; sh >>= 1) {
        const int o = __shfl_xor(wave_lim, sh);
        wave_lim = o > wave_lim ? o : wave_lim;
    }
    wave_lim = __builtin_amdgcn_readfirstlane(wave_lim);

    // ---- Q fragments: B operand of S^T = K Q^T; lane holds Q[col][32 s + 8 kq .. +8] ----
    f16x8 qf[KSTEPS];
    {
        const half_t* qp = (const half_t*)a.query + (q_row0 + pos_c) * a.query_stride_s + (int64_t)h * D + 8 * kq;
#pragma unroll
        for (int s = 0; s < KSTEPS; ++s) qf[s] = *(const f16x8*)(qp + 32 * s);
    }

    f32x4 o_acc[CT];
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) o_acc[ct] = f32x4{0.f, 0.f, 0.f, 0.f};
    float m_run = kNegBig, l_run = 0.f;
    const half_t* mask_row = nullptr;
    float slope = 0.f;
    if (EXTRA) {
        if (a.attn_mask)
            mask_row = (const half_t*)a.attn_mask + (int64_t)h * a.mask_stride_h + (q_row0 + pos_c) * a.mask_stride_s + a.kvstarts[b];
        if (a.alibi_slopes) slope = a.alibi_slopes[h];
    }

    // ---- global -> register staging of one tile's raw bytes ----
    const int64_t table_base = PAGED ? (int64_t)b * a.cachestarts_stride_b : (int64_t)b;
    u32x2 k_raw[UNITS], v_raw[UNITS];
    half_t k_sc[UNITS], v_sc[UNITS];
    u32x4 k16[UNITS], v16[UNITS];
    // a tile of 32 tokens starts at a multiple of 32, so it lies inside one 128-token page
    auto tile_row = [&](int tile) -> int64_t {
        int t_base = tile * kBN16;
        if (t_base > kvlen - 1) t_base = kvlen > 0 ? kvlen - 1 : 0;
        if (KV16) return q_row0 + t_base;
        if (PAGED) return cachestarts[table_base + (t_base >> 7)] + (t_base & (kPage - 1));
        return cachestarts[table_base] + t_base;
    };
    auto load_tile = [&](int tile) {
        const int64_t row = tile_row(tile);
        const int left = kvlen - 1 - tile * kBN16; // offset of the sequence's last token inside this tile
#pragma unroll
        for (int u = 0; u < UNITS; ++u) {
            if (!u_on[u]) continue;
            // tokens beyond the sequence re-read its last token (masked later)
            const uint32_t t = (uint32_t)(u_t[u] < left ? u_t[u] : (left > 0 ? left : 0));
            if (KV16) {
                const half_t* bk = (const half_t*)a.current_key + row * a.key_stride_s + (int64_t)kvh * D;
                const half_t* bv = (const half_t*)a.current_value + row * a.value_stride_s + (int64_t)kvh * D;
                k16[u] = *(const u32x4*)(bk + t * kstride16 + 8 * u_g[u]);
                v16[u] = *(const u32x4*)(bv + t * vstride16 + 8 * u_g[u]);
            } else {
                const int64_t boff = row * a.cache_stride_s;
                const uint32_t off = t * stride_s32 + 8 * (uint32_t)u_g[u];
                k_raw[u] = *(const u32x2*)(cache_k + boff + off);
                k_sc[u] = (scale_k + (boff >> 3))[off >> 3];
                v_raw[u] = *(const u32x2*)(cache_v + boff + off);
                v_sc[u] = (scale_v + (boff >> 3))[off >> 3];
            }
        }
    };
    auto split_store = [&](half_t* dst, half_t* dst_lo, const u32x2 raw, const half_t scl) {
        const half2_t sc = {scl, scl};
        const uint32_t f0 = raw[0] ^ kFlipSigns, f1 = raw[1] ^ kFlipSigns;
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
        *(u32x4*)dst = w;
        *(u32x4*)dst_lo = wl;
    };
    auto store_tile = [&](int buf) {
        half_t* const sK = smem + buf * TILE_HALVES;
        half_t* const sKlo = sK + K_HALVES;
        half_t* const sV = KV16 ? sKlo : sKlo + K_HALVES;
        half_t* const sVlo = sV + V_HALVES;
#pragma unroll
        for (int u = 0; u < UNITS; ++u) {
            if (!u_on[u]) continue;
            half_t* const dk = &sK[u_t[u] * K_STRIDE + 8 * u_g[u]];
            half_t* const dv = &sV[u_t[u] * V_STRIDE + 8 * u_g[u]];
            if (KV16) {
                *(u32x4*)dk = k16[u];
                *(u32x4*)dv = v16[u];
            } else {
                split_store(dk, &sKlo[u_t[u] * K_STRIDE + 8 * u_g[u]], k_raw[u], k_sc[u]);
                split_store(dv, &sVlo[u_t[u] * V_STRIDE + 8 * u_g[u]], v_raw[u], v_sc[u]);
            }
        }
    };

    __syncthreads(); // the previous item's last tile has been read by every wave
    if (n_tiles > 0) {
        load_tile(0);
        store_tile(0);
        if (n_tiles > 1) load_tile(1);
        __syncthreads();
    }

    for (int tile = 0; tile < n_tiles; ++tile) {
        const int buf = tile & 1;
        // the next tile into the other buffer (every wave is past its reads of it since the barrier that ended the
        // previous iteration), and the raw bytes of the tile after next into the freed registers
        if (tile + 1 < n_tiles) store_tile(buf ^ 1);
        if (tile + 2 < n_tiles) load_tile(tile + 2);

        const int t_base = tile * kBN16;
        if (t_base < wave_lim) { // a wave whose columns end before this tile only helps to stage it
            const half_t* const sK = smem + buf * TILE_HALVES;
            const half_t* const sKlo = sK + K_HALVES;
            const half_t* const sV = KV16 ? sKlo : sKlo + K_HALVES;
            const half_t* const sVlo = sV + V_HALVES;

            // ---- S^T: two tiles of 16 tokens ----
            f32x4 sacc[2];
#pragma unroll
            for (int mb = 0; mb < 2; ++mb) {
                sacc[mb] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int s = 0; s < KSTEPS; ++s) {
                    const f16x8 fh = *(const f16x8*)&sK[k_frag_off + 16 * mb * K_STRIDE + 32 * s];
                    if (!KV16) {
                        const f16x8 fl = *(const f16x8*)&sKlo[k_frag_off + 16 * mb * K_STRIDE + 32 * s];
                        sacc[mb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(fl, qf[s], sacc[mb], 0, 0, 0);
                    }
                    sacc[mb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(fh, qf[s], sacc[mb], 0, 0, 0);
                }
            }

            // ---- softmax: element j of tile mb is token t_base + 16 mb + 4 kq + j ----
            float v[8];
            float mx = kNegBig;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const int t = t_base + 16 * (e >> 2) + 4 * kq + (e & 3);
                float x = -INFINITY;
                if (t < lim) {
                    if (EXTRA) {
                        float add = 0.f;
                        if (mask_row) add = (float)mask_row[t];
                        if (a.alibi_slopes) add += a.is_causal ? slope * (float)t : -slope * fabsf((float)(pos_c + kvlen - qlen - t));
                        x = __builtin_fmaf(sacc[e >> 2][e & 3], sm_scale, add * kLog2e);
                    } else {
                        x = sacc[e >> 2][e & 3] * sm_scale;
                    }
                }
                v[e] = x;
                mx = fmaxf(mx, x);
            }
            {
                // across the four quarters of the wave with the vector unit's lane swaps (no data-share permute, which
                // would wait for the fragment reads queued behind it)
                const u32x2 rows = __builtin_amdgcn_permlane16_swap(bitcast<uint32_t>(mx), bitcast<uint32_t>(mx), false, false);
                mx = fmaxf(bitcast<float>(rows[0]), bitcast<float>(rows[1]));
                const u32x2 both = __builtin_amdgcn_permlane32_swap(bitcast<uint32_t>(mx), bitcast<uint32_t>(mx), false, false);
                mx = fmaxf(bitcast<float>(both[0]), bitcast<float>(both[1]));
            }
            const float m_new = fmaxf(m_run, mx);
            if (__builtin_amdgcn_ballot_w64(m_new > m_run) != 0) { // rare after the first tiles (wave-uniform)
                const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
                l_run *= alpha;
#pragma unroll
                for (int ct = 0; ct < CT; ++ct) o_acc[ct] *= alpha;
                m_run = m_new;
            }
            // p = 2^(logit - max) * 2^14 as hi + lo halves (hi rounded toward zero, lo the exact remainder)
            const float bias = kPShift - m_run;
            f16x8 ph, pl;
#pragma unroll
            for (int e = 0; e < 8; e += 2) {
                const float q0 = __builtin_amdgcn_exp2f(v[e] + bias), q1 = __builtin_amdgcn_exp2f(v[e + 1] + bias);
                l_run += q0 + q1;
                const half2_t h2 = bitcast<half2_t>(__builtin_amdgcn_cvt_pkrtz(q0, q1));
                const half2_t l2 = bitcast<half2_t>(__builtin_amdgcn_cvt_pkrtz(sub_half_lo(q0, h2), sub_half_hi(q1, h2)));
                ph[e] = h2.x;
                ph[e + 1] = h2.y;
                pl[e] = l2.x;
                pl[e + 1] = l2.y;
            }

            // ---- O^T += V^T P^T: channel tile ct, the lane's 8 tokens from two transposing reads ----
            typedef short s16x4 __attribute__((ext_vector_type(4)));
            typedef __attribute__((address_space(3))) s16x4* lds_s16x4_ptr;
            auto read_vt = [&](const half_t* base, int ct) -> f16x8 {
                const half_t* p = base + v_frag_off + 16 * ct;
                const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(p));
                const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(p + 16 * V_STRIDE));
                return bitcast<f16x8>(__builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
            };
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) {
                const f16x8 vh = read_vt(sV, ct);
                if (!KV16) {
                    const f16x8 vl = read_vt(sVlo, ct);
                    o_acc[ct] = __builtin_amdgcn_mfma_f32_16x16x32_f16(vl, ph, o_acc[ct], 0, 0, 0);
                }
                o_acc[ct] = __builtin_amdgcn_mfma_f32_16x16x32_f16(vh, pl, o_acc[ct], 0, 0, 0);
                o_acc[ct] = __builtin_amdgcn_mfma_f32_16x16x32_f16(vh, ph, o_acc[ct], 0, 0, 0);
            }
        }
        __syncthreads(); // tile + 1 is complete in the other buffer; this buffer may be overwritten
    }

    // ---- normalise and store: element j of tile ct <-> channel 16 ct + 4 kq + j ----
    float l_tot = l_run + __shfl_xor(l_run, 16);
    l_tot += __shfl_xor(l_tot, 32);
    const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
    if (col_on) {
        half_t* op = (half_t*)a.output + (q_row0 + pos) * a.output_stride_s + (int64_t)h * D + 4 * kq;
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) {
            f16x4 w;
#pragma unroll
            for (int e = 0; e < 4; ++e) w[e] = (half_t)(o_acc[ct][e] * inv);
            *(f16x4*)(op + 16 * ct) = w;
        }
    }
    } // items
}

template <int D, int SRC>
constexpr size_t prefill_lds_bytes()
{
    // int8 source: K hi/lo tiles + V hi/lo tiles (above the 64 KB static limit for D = 128, hence dynamic);
    // fp16 source: one K tile and one V tile; two buffers of each.  The epilogue's staging (eight waves x 32 rows and
    // their offsets) starts where the second buffer starts and may reach beyond it.
    constexpr size_t tiles = 2 * (SRC == 2 ? 1 : 2) * kBN * (PrefillTile<D>::K_STRIDE + PrefillTile<D>::V_STRIDE) * sizeof(half_t);
    constexpr size_t with_epilogue = (kEpilogueBase<D, SRC>() + 8 * (32 * (D + 8) + 32 * 4)) * sizeof(half_t);
    return tiles > with_epilogue ? tiles : with_epilogue;
}

template <int D, int SRC, bool EXTRA>
static DeviceMask& prefill_variant_ready()
{
    static DeviceMask ready{0};
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

template <int D, int SRC>
constexpr size_t prefill16_lds_bytes()
{
    return 2 * (SRC == 2 ? 1 : 2) * kBN16 * (PrefillTile16<D>::K_STRIDE + PrefillTile16<D>::V_STRIDE) * sizeof(half_t);
}

template <int D, int SRC, bool EXTRA>
static DeviceMask& prefill16_variant_ready()
{
    static DeviceMask ready{0};
    return ready;
}

template <int D, int SRC, bool EXTRA>
static int launch_prefill16_variant(const PrefillLaunch& a, dim3 grid, hipStream_t stream)
{
    constexpr size_t lds_bytes = prefill16_lds_bytes<D, SRC>();
    if (int rc = ensure_dynamic_lds((const void*)prefill_attention16_kernel<D, SRC, EXTRA>, (int)lds_bytes, stream,
                                    prefill16_variant_ready<D, SRC, EXTRA>()))
        return rc;
    hipLaunchKernelGGL((prefill_attention16_kernel<D, SRC, EXTRA>), grid, dim3(kPrefillThreads), lds_bytes, stream, a);
    return kLaunchOk;
}

template <int D>
static int launch_prefill16_d(const PrefillLaunch& a, hipStream_t stream)
{
    const int G = (int)(a.num_heads / a.num_kv_heads);
    if (G > kCols16) return kLaunchNoKernel;
    const int ppw = kCols16 / G > 0 ? kCols16 / G : 1;
    int64_t items = a.prefill_batches * ((a.max_seqlen + ppw - 1) / ppw);
    if (a.query_rows > 0 && a.prefill_batches <= 64 * kPickSlots) {
        const int64_t by_rows = a.query_rows / ppw + a.prefill_batches;
        if (by_rows < items) items = by_rows;
    }
    if (items * a.num_kv_heads > 0x7fffffff) return kLaunchNoKernel;
    const dim3 grid((unsigned)(items * a.num_kv_heads), 1, 1);
    const bool extra = a.attn_mask != nullptr || a.alibi_slopes != nullptr;
    const int src = a.current_key ? 2 : (a.cache_mode == 1 ? 0 : 1);
    if (extra) {
        if (src == 0) return launch_prefill16_variant<D, 0, true>(a, grid, stream);
        if (src == 1) return launch_prefill16_variant<D, 1, true>(a, grid, stream);
        return launch_prefill16_variant<D, 2, true>(a, grid, stream);
    }
    if (src == 0) return launch_prefill16_variant<D, 0, false>(a, grid, stream);
    if (src == 1) return launch_prefill16_variant<D, 1, false>(a, grid, stream);
    return launch_prefill16_variant<D, 2, false>(a, grid, stream);
}

int launch_prefill(const PrefillLaunch& a, hipStream_t stream)
{
    switch (a.head_dim) {
        case 64: return a.num_heads / a.num_kv_heads > kCols ? kLaunchNoKernel : launch_prefill_d<64>(a, stream);
        case 128: return a.num_heads / a.num_kv_heads > kCols ? kLaunchNoKernel : launch_prefill_d<128>(a, stream);
        case 96: return a.num_heads / a.num_kv_heads > kCols ? kLaunchNoKernel : launch_prefill_d<96>(a, stream);
        case 256: return launch_prefill16_d<256>(a, stream);
        default: return kLaunchNoKernel;
    }
}

template <int D, int SRC, bool EXTRA>
static int init_prefill_variant()
{
    return set_dynamic_lds_once((const void*)prefill_attention_kernel<D, SRC, EXTRA>, (int)prefill_lds_bytes<D, SRC>(),
                                prefill_variant_ready<D, SRC, EXTRA>());
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
template <int D, int SRC, bool EXTRA>
static int init_prefill16_variant()
{
    return set_dynamic_lds_once((const void*)prefill_attention16_kernel<D, SRC, EXTRA>, (int)prefill16_lds_bytes<D, SRC>(),
                                prefill16_variant_ready<D, SRC, EXTRA>());
}
template <int D>
static int init_prefill16_d()
{
    if (int rc = init_prefill16_variant<D, 0, false>()) return rc;
    if (int rc = init_prefill16_variant<D, 0, true>()) return rc;
    if (int rc = init_prefill16_variant<D, 1, false>()) return rc;
    if (int rc = init_prefill16_variant<D, 1, true>()) return rc;
    if (int rc = init_prefill16_variant<D, 2, false>()) return rc;
    return init_prefill16_variant<D, 2, true>();
}
int init_prefill_kernels()
{
    if (int rc = init_prefill_d<64>()) return rc;
    if (int rc = init_prefill_d<96>()) return rc;
    if (int rc = init_prefill_d<128>()) return rc;
    return init_prefill16_d<256>();
}

} // namespace pmxhip
