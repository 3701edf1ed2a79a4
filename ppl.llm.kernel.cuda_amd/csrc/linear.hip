// Output projection behind the attention: output(M, N) = input(M, K) * weight(N, K)^T + bias, fp16 in and out,
// fp32 accumulate -- the single-rank case of the reference's row_parallel_linear
// (src/ppl/kernel/llm/cuda/pmx/row_parallel_linear.cu:25-110: one cublasLt GEMM, then an all-reduce only when the
// communicator has more than one rank).
//
// At a decode step M is the number of sequences (tens to a few hundred) and the call is bound by streaming the
// weights: K * N * 2 bytes, each read once.  Decomposition (this file's own): a workgroup owns 16 output columns
// (16 weight rows) and up to 128 input rows, so with N = 4096 the 256 workgroups each stream 128 KB of weights.
// Both operands are contiguous along K, which is the k dimension of v_mfma_f32_16x16x32_f16 for both of its
// inputs: a lane loads 16 bytes of a weight row (A: 16 columns x 32 k) and 16 bytes of each of eight input rows
// (B: 32 k x 16 rows), no transposition anywhere; the accumulator then holds four consecutive output columns of
// one row per lane.  The eight waves of the workgroup take the 32-wide k steps in turn (adjacent 64-byte pieces
// of a weight row: a 512-byte run per row and round), keep the weight requests four steps ahead and the input
// requests two, and add their partial tiles through LDS at the end, in a fixed order: the result does not depend
// on timing.  The input (M * K * 2 bytes, 1 MB at M = 128) is read by every workgroup and comes from L2.
#include "device_common.h"
#include "launch_params.h"

namespace pmxhip {

namespace {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));

constexpr int kLinWaves = 8;
constexpr int kLinThreads = 64 * kLinWaves;
constexpr int kLinCols = 16;   // output columns per workgroup
constexpr int kLinRows = 128;  // input rows per workgroup
constexpr int kLinMB = kLinRows / 16;
constexpr int kLinKStep = 32;
constexpr int kWDepth = 4, kADepth = 2;

} // namespace

__global__ __launch_bounds__(kLinThreads) void skinny_linear_kernel(const LinearLaunch a)
{
    __shared__ __attribute__((aligned(16))) float s_part[kLinWaves][kLinRows][kLinCols]; // 64 KB
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r16 = lane & 15;  // weight row (output column) / input row within a 16-row block
    const int kq = lane >> 4;   // which 8 of the 32 k of a step
    const int64_t n0 = (int64_t)blockIdx.x * kLinCols;
    const int64_t m0 = (int64_t)blockIdx.y * kLinRows;
    const int ksteps = (int)(a.k / kLinKStep);
    const int my_steps = (ksteps - wave + kLinWaves - 1) / kLinWaves; // steps wave, wave + 8, ...

    const half_t* wp = (const half_t*)a.weight + (n0 + r16) * a.weight_stride + 8 * kq;
    const half_t* ip[kLinMB];
#pragma unroll
    for (int mb = 0; mb < kLinMB; ++mb) {
        int64_t m = m0 + 16 * mb + r16;
        if (m > a.m - 1) m = a.m - 1; // rows beyond the batch re-read its last row; their results are not stored
        ip[mb] = (const half_t*)a.input + m * a.input_stride + 8 * kq;
    }

    f32x4 acc[kLinMB];
#pragma unroll
    for (int mb = 0; mb < kLinMB; ++mb) acc[mb] = f32x4{0.f, 0.f, 0.f, 0.f};

    f16x8 wf[kWDepth];
    f16x8 af[kADepth][kLinMB];
    auto k_of = [&](int i) { return (int64_t)(i * kLinWaves + wave) * kLinKStep; };
    auto load_w = [&](int i, f16x8& dst) {
        const int ic = i < my_steps ? i : my_steps - 1; // past the end: a harmless repeat of the last step
        dst = __builtin_nontemporal_load((const f16x8*)(wp + k_of(ic))); // every weight byte is used once
    };
    auto load_a = [&](int i, f16x8* dst) {
        const int ic = i < my_steps ? i : my_steps - 1;
#pragma unroll
        for (int mb = 0; mb < kLinMB; ++mb) dst[mb] = *(const f16x8*)(ip[mb] + k_of(ic));
    };
    if (my_steps > 0) {
#pragma unroll
        for (int d = 0; d < kWDepth; ++d) load_w(d, wf[d]);
#pragma unroll
        for (int d = 0; d < kADepth; ++d) load_a(d, af[d]);
        // the rings are indexed with compile-time constants: the loop runs over groups of kWDepth steps
        for (int i0 = 0; i0 < my_steps; i0 += kWDepth) {
#pragma unroll
            for (int d = 0; d < kWDepth; ++d) {
                const int i = i0 + d;
                if (i < my_steps) {
                    const f16x8 w = wf[d];
                    f16x8 cur[kLinMB];
#pragma unroll
                    for (int mb = 0; mb < kLinMB; ++mb) cur[mb] = af[d % kADepth][mb];
                    load_w(i + kWDepth, wf[d]);
                    load_a(i + kADepth, af[d % kADepth]);
#pragma unroll
                    for (int mb = 0; mb < kLinMB; ++mb)
                        acc[mb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(w, cur[mb], acc[mb], 0, 0, 0);
                }
            }
        }
    }

    // accumulator element e of block mb: row 16 mb + r16, column 4 kq + e
#pragma unroll
    for (int mb = 0; mb < kLinMB; ++mb) *(f32x4*)&s_part[wave][16 * mb + r16][4 * kq] = acc[mb];
    __syncthreads();
    // one thread per (row, four columns): the eight partial tiles are added in wave order
    {
        const int row = tid >> 2, c4 = (tid & 3) * 4;
        f32x4 sum = *(const f32x4*)&s_part[0][row][c4];
#pragma unroll
        for (int w = 1; w < kLinWaves; ++w) sum += *(const f32x4*)&s_part[w][row][c4];
        if (a.bias) {
            const f16x4 b = *(const f16x4*)((const half_t*)a.bias + n0 + c4);
#pragma unroll
            for (int e = 0; e < 4; ++e) sum[e] += (float)b[e];
        }
        if (m0 + row < a.m) {
            f16x4 o;
#pragma unroll
            for (int e = 0; e < 4; ++e) o[e] = (half_t)sum[e];
            *(f16x4*)((half_t*)a.output + (m0 + row) * a.output_stride + n0 + c4) = o;
        }
    }
}

// ---- the decode-step form: 64 output columns per workgroup, K split over workgroups ------------------------------
// What bounds the kernel above at M = 128 is not the weight stream but the input: every workgroup reads all of it
// (1 MB through a CU's 64-byte-per-clock path to L2: 8 us, five times the time of its 128 KB of weights; measured
// 42 us for 4096 x 4096).  Here a workgroup owns 64 columns, so the input is read N / 64 times instead of N / 16,
// and the k range is split over `splits` workgroups to keep every CU busy: 4096 x 4096 on 256 CUs = 64 column
// blocks x 8 k ranges, each with 64 KB of weights and 128 KB of input, two workgroups per CU.  A wave owns 16 of the 64 columns and
// requests its whole weight slice (16 rows x up to 512 k = 16 fragments = 64 registers) before anything else, so
// a CU has all its weight bytes in flight at once; the input rows pass through LDS in stages of 64 k (one
// coalesced copy per workgroup, read back as fragments by all four waves).  With splits > 1 the float32 partial
// tiles go to the workspace and linear_reduce_kernel adds them in a fixed order.
namespace {
constexpr int kSplitCols = 64;
constexpr int kSplitThreads = 256;
constexpr int kSplitStage = 64;             // k per LDS stage
constexpr int kSplitRowHalves = kSplitStage + 8; // +16 bytes: the fragment reads of 16 rows cover all banks
constexpr int kSplitChunk = 512;            // k per register-resident weight slice
constexpr int kSplitWFrags = kSplitChunk / kLinKStep;
} // namespace

__global__ __launch_bounds__(kSplitThreads) void split_linear_kernel(const LinearLaunch a, const int splits, float* __restrict__ partial)
{
    __shared__ __attribute__((aligned(16))) half_t s_in[2][kLinRows][kSplitRowHalves]; // 36 KB
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r16 = lane & 15;
    const int kq = lane >> 4;
    const int64_t n0 = (int64_t)blockIdx.x * kSplitCols + 16 * wave;
    const int64_t m0 = (int64_t)blockIdx.z * kLinRows;
    const int64_t k_len = a.k / splits;
    const int64_t k_begin = (int64_t)blockIdx.y * k_len;

    // the copy of an input stage: thread t moves 16 bytes of row (t / 8) + 32 j, k piece t % 8, j = 0..3
    const int c_row = tid >> 3, c_k = (tid & 7) * 8;
    const half_t* cp[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        int64_t m = m0 + c_row + 32 * j;
        if (m > a.m - 1) m = a.m - 1; // rows beyond the batch re-read its last row; their results are not stored
        cp[j] = (const half_t*)a.input + m * a.input_stride + c_k;
    }
    const half_t* wp = (const half_t*)a.weight + (n0 + r16) * a.weight_stride + 8 * kq;

    f32x4 acc[kLinMB];
#pragma unroll
    for (int mb = 0; mb < kLinMB; ++mb) acc[mb] = f32x4{0.f, 0.f, 0.f, 0.f};

    for (int64_t kc = 0; kc < k_len; kc += kSplitChunk) {
        const int64_t k0 = k_begin + kc;
        const int chunk = (int)(k_len - kc < kSplitChunk ? k_len - kc : kSplitChunk); // multiple of 64
        const int stages = chunk / kSplitStage;
        // this wave's weight slice of the chunk, all of it in flight at once (streamed: every byte is used once)
        f16x8 wf[kSplitWFrags];
#pragma unroll
        for (int i = 0; i < kSplitWFrags; ++i) {
            const int ic = i * kLinKStep < chunk ? i : 0;
            wf[i] = __builtin_nontemporal_load((const f16x8*)(wp + k0 + ic * kLinKStep));
        }
        u32x4 stage_regs[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) stage_regs[j] = *(const u32x4*)(cp[j] + k0);
        __syncthreads(); // the previous chunk's last stage has been read
#pragma unroll
        for (int j = 0; j < 4; ++j) *(u32x4*)&s_in[0][c_row + 32 * j][c_k] = stage_regs[j];
        __syncthreads();
#pragma unroll
        for (int st2 = 0; st2 < kSplitChunk / kSplitStage; st2 += 2) {
#pragma unroll
            for (int par = 0; par < 2; ++par) {
                const int st = st2 + par;
                if (st < stages) {
                    if (st + 1 < stages) {
#pragma unroll
                        for (int j = 0; j < 4; ++j) stage_regs[j] = *(const u32x4*)(cp[j] + k0 + (st + 1) * kSplitStage);
                    }
#pragma unroll
                    for (int h = 0; h < 2; ++h) {
                        f16x8 bf[kLinMB];
#pragma unroll
                        for (int mb = 0; mb < kLinMB; ++mb) bf[mb] = *(const f16x8*)&s_in[par][16 * mb + r16][32 * h + 8 * kq];
#pragma unroll
                        for (int mb = 0; mb < kLinMB; ++mb)
                            acc[mb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(wf[2 * st + h], bf[mb], acc[mb], 0, 0, 0);
                    }
                    if (st + 1 < stages) {
#pragma unroll
                        for (int j = 0; j < 4; ++j) *(u32x4*)&s_in[par ^ 1][c_row + 32 * j][c_k] = stage_regs[j];
                    }
                    __syncthreads(); // stage st + 1 is complete; stage st may be overwritten two stages on
                }
            }
        }
    }

    // accumulator element e of block mb: row 16 mb + r16, column n0 + 4 kq + e
    if (splits > 1) {
        float* part = partial + ((int64_t)blockIdx.y * a.m + m0) * a.n + n0 + 4 * kq;
#pragma unroll
        for (int mb = 0; mb < kLinMB; ++mb)
            if (m0 + 16 * mb + r16 < a.m) *(f32x4*)(part + (int64_t)(16 * mb + r16) * a.n) = acc[mb];
    } else {
        f32x4 bias = {0.f, 0.f, 0.f, 0.f};
        if (a.bias) {
            const f16x4 b = *(const f16x4*)((const half_t*)a.bias + n0 + 4 * kq);
#pragma unroll
            for (int e = 0; e < 4; ++e) bias[e] = (float)b[e];
        }
#pragma unroll
        for (int mb = 0; mb < kLinMB; ++mb) {
            const int64_t row = m0 + 16 * mb + r16;
            if (row < a.m) {
                f16x4 o;
#pragma unroll
                for (int e = 0; e < 4; ++e) o[e] = (half_t)(acc[mb][e] + bias[e]);
                *(f16x4*)((half_t*)a.output + row * a.output_stride + n0 + 4 * kq) = o;
            }
        }
    }
}

// ---- the same decomposition without LDS staging: a wave owns a k range, not a column range ------------------------
// In the kernel above the input passes through LDS in stages of 64 k behind a barrier each, one stage ahead: a
// workgroup's time is then eight L2 latencies in a row, not its bytes.  Here the four waves of a workgroup split the
// workgroup's k range between them (in turns of 64 k, so that the four waves together read 512-byte runs of a row)
// and each computes all 64 columns over its k: the weight fragments and the input fragments of a wave are then its
// own -- both come straight from memory in the MFMA operand layout (16 bytes of a row per lane), nothing is shared,
// and there is no barrier before the end.  A weight fragment serves MT row blocks and an input fragment four column
// blocks, as before.  A turn is 32 k (4 weight and MT input fragments); a wave requests a turn three turns ahead
// of its products, so with MT = 8 it has up to 36 KB on its way (one workgroup per CU, up to 512 registers per
// lane).  The four partial tiles of a workgroup are added pairwise through LDS in a fixed order.
template <int MT>
__global__ __launch_bounds__(256, 1) void wavek_linear_kernel(const LinearLaunch a, const int splits, float* __restrict__ partial)
{
    constexpr int kTiles = 4 * MT;
    __shared__ __attribute__((aligned(16))) f32x4 s_red[2][kTiles][64]; // MT = 8: 64 KB
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int r16 = lane & 15;
    const int kq = lane >> 4;
    const int64_t n0 = (int64_t)blockIdx.x * 64;
    const int64_t m0 = (int64_t)blockIdx.z * (16 * MT);
    const int64_t k_len = a.k / splits; // a multiple of 512: every wave has the same, even number of turns
    const int64_t k_begin = (int64_t)blockIdx.y * k_len;
    const int turns = (int)(k_len >> 8);

    const half_t* wp = (const half_t*)a.weight + (n0 + r16) * a.weight_stride + k_begin + 64 * wave + 8 * kq;
    const int64_t w16 = 16 * a.weight_stride;
    const half_t* ip[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        int64_t m = m0 + 16 * mt + r16;
        if (m > a.m - 1) m = a.m - 1; // rows beyond the batch re-read its last row; their results are not stored
        ip[mt] = (const half_t*)a.input + m * a.input_stride + k_begin + 64 * wave + 8 * kq;
    }

    // a turn: 64 k (one 128-byte line of each row, both halves requested together) of the wave's 64 columns and
    // 16 MT rows
    struct Turn {
        f16x8 w[2][4];
        f16x8 in[2][MT];
    };
    Turn r0, r1;
    auto request = [&](int t, Turn& dst) {
        const int64_t k = (int64_t)t * 256;
#pragma unroll
        for (int nt = 0; nt < 4; ++nt)
#pragma unroll
            for (int h = 0; h < 2; ++h) dst.w[h][nt] = __builtin_nontemporal_load((const f16x8*)(wp + nt * w16 + k + 32 * h));
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int h = 0; h < 2; ++h) dst.in[h][mt] = *(const f16x8*)(ip[mt] + k + 32 * h);
        __builtin_amdgcn_sched_barrier(0); // the requests stay where they are written: ahead of the products below
    };

    f32x4 acc[4][MT];
#pragma unroll
    for (int nt = 0; nt < 4; ++nt)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[nt][mt] = f32x4{0.f, 0.f, 0.f, 0.f};

    auto products = [&](const Turn& u) {
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int nt = 0; nt < 4; ++nt)
#pragma unroll
                for (int mt = 0; mt < MT; ++mt)
                    acc[nt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(u.w[h][nt], u.in[h][mt], acc[nt][mt], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
    };

    // Straight-line code between the loop's branches, so that the waits the compiler places count exactly the
    // requests that may still be on their way; the last two turns are peeled because they have nothing to request.
    request(0, r0);
    request(1, r1);
    int t = 0;
    for (; t + 4 <= turns; t += 2) {
        products(r0);
        request(t + 2, r0);
        products(r1);
        request(t + 3, r1);
    }
    products(r0);
    products(r1);

    // (wave 0 + wave 2) + (wave 1 + wave 3): a lane reads back the slots it would have written itself
    if (wave >= 2) {
#pragma unroll
        for (int nt = 0; nt < 4; ++nt)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) s_red[wave - 2][nt * MT + mt][lane] = acc[nt][mt];
    }
    __syncthreads();
    if (wave < 2) {
#pragma unroll
        for (int nt = 0; nt < 4; ++nt)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) acc[nt][mt] += s_red[wave][nt * MT + mt][lane];
    }
    __syncthreads();
    if (wave == 1) {
#pragma unroll
        for (int nt = 0; nt < 4; ++nt)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) s_red[0][nt * MT + mt][lane] = acc[nt][mt];
    }
    __syncthreads();
    if (wave != 0) return;
#pragma unroll
    for (int nt = 0; nt < 4; ++nt)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[nt][mt] += s_red[0][nt * MT + mt][lane];

    // accumulator element e of tile (nt, mt): row m0 + 16 mt + r16, column n0 + 16 nt + 4 kq + e
    if (splits > 1) {
        float* part = partial + ((int64_t)blockIdx.y * a.m + m0) * a.n + n0 + 4 * kq;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            if (m0 + 16 * mt + r16 < a.m) {
#pragma unroll
                for (int nt = 0; nt < 4; ++nt) *(f32x4*)(part + (int64_t)(16 * mt + r16) * a.n + 16 * nt) = acc[nt][mt];
            }
        }
    } else {
#pragma unroll
        for (int nt = 0; nt < 4; ++nt) {
            f32x4 bias = {0.f, 0.f, 0.f, 0.f};
            if (a.bias) {
                const f16x4 b = *(const f16x4*)((const half_t*)a.bias + n0 + 16 * nt + 4 * kq);
#pragma unroll
                for (int e = 0; e < 4; ++e) bias[e] = (float)b[e];
            }
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                const int64_t row = m0 + 16 * mt + r16;
                if (row < a.m) {
                    f16x4 o;
#pragma unroll
                    for (int e = 0; e < 4; ++e) o[e] = (half_t)(acc[nt][mt][e] + bias[e]);
                    *(f16x4*)((half_t*)a.output + row * a.output_stride + n0 + 16 * nt + 4 * kq) = o;
                }
            }
        }
    }
}

// output = half(sum over the k ranges of the partial tiles, in range order, + bias); four columns per thread
__global__ __launch_bounds__(256) void linear_reduce_kernel(const LinearLaunch a, const int splits, const float* __restrict__ partial)
{
    const int64_t quads = a.n >> 2;
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= a.m * quads) return;
    const int64_t row = i / quads, c4 = (i - row * quads) * 4;
    f32x4 sum = *(const f32x4*)(partial + row * a.n + c4);
    for (int s = 1; s < splits; ++s) sum += *(const f32x4*)(partial + ((int64_t)s * a.m + row) * a.n + c4);
    if (a.bias) {
        const f16x4 b = *(const f16x4*)((const half_t*)a.bias + c4);
#pragma unroll
        for (int e = 0; e < 4; ++e) sum[e] += (float)b[e];
    }
    f16x4 o;
#pragma unroll
    for (int e = 0; e < 4; ++e) o[e] = (half_t)sum[e];
    *(f16x4*)((half_t*)a.output + row * a.output_stride + c4) = o;
}

// Row blocks of 16 a workgroup of wavek_linear_kernel takes: the smallest of 1, 2, 4, 8 that covers m, else 8
static int wavek_row_blocks(int64_t m)
{
    return m > 64 ? 8 : m > 32 ? 4 : m > 16 ? 2 : 1;
}

// k ranges for wavek_linear_kernel: the largest power of two up to 16 that still gives every workgroup a CU of its
// own in one round, each range a multiple of 512 (four turns of 32 k for each of four waves); 0 when the shape is
// not for that kernel
static int wavek_splits(int64_t m, int64_t n, int64_t k, int compute_units)
{
    if (n % 64 != 0 || k % 512 != 0) return 0;
    const int64_t rows = 16 * wavek_row_blocks(m);
    const int64_t wgs = (n / 64) * ((m + rows - 1) / rows);
    const int64_t cus = compute_units > 0 ? compute_units : 256;
    int s = 1;
    while (s < 16 && wgs * s * 2 <= cus && k % (s * 2 * 512) == 0) s *= 2;
    return s;
}

// k ranges for split_linear_kernel: as many as give every CU two workgroups, a power of two up to 16, each a multiple
// of 64 and at least 256 long; 0 when the shape is for the general kernel (N not in 64s, K not in 64s)
int linear_splits(int64_t m, int64_t n, int64_t k, int compute_units)
{
    if (n % kSplitCols != 0 || k % kSplitStage != 0) return 0;
    const int64_t wgs = (n / kSplitCols) * ((m + kLinRows - 1) / kLinRows);
    int s = 1;
    // two workgroups per CU: one's waits for its input stages are the other's products
    while (s < 16 && wgs * s * 2 <= 2 * (compute_units > 0 ? compute_units : 256) && k % (s * 2 * kSplitStage) == 0 && k / (s * 2) >= 256) s *= 2;
    return s;
}

int64_t linear_workspace_bytes(int64_t m, int64_t n, int64_t k, int compute_units)
{
    int s = wavek_splits(m, n, k, compute_units);
    if (s == 0) s = linear_splits(m, n, k, compute_units);
    return s > 1 ? (int64_t)s * m * n * (int64_t)sizeof(float) : 0;
}

int launch_linear(const LinearLaunch& a, int compute_units, void* workspace, int64_t workspace_bytes, hipStream_t stream)
{
    if (a.m <= 0 || a.n <= 0) return kLaunchOk;
    if (a.n % kLinCols != 0 || a.k % kLinKStep != 0 || a.k <= 0) return kLaunchNoKernel;
    const int64_t mblocks = (a.m + kLinRows - 1) / kLinRows;
    if (a.n / kLinCols > 0x7fffffff || mblocks > 65535) return kLaunchNoKernel;
    // as many k ranges as the workspace holds partial tiles for; none: one k range per column block (fewer workgroups
    // than CUs at decode sizes)
    if (!workspace || (reinterpret_cast<uintptr_t>(workspace) & 15u)) workspace_bytes = 0;
    auto fit = [&](int splits) {
        while (splits > 1 && workspace_bytes < (int64_t)splits * a.m * a.n * (int64_t)sizeof(float)) splits /= 2;
        return splits;
    };
    auto reduce = [&](int splits) {
        if (splits <= 1) return;
        const int64_t threads = a.m * (a.n >> 2);
        hipLaunchKernelGGL(linear_reduce_kernel, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, stream, a, splits,
                           (const float*)workspace);
    };
    int splits = fit(wavek_splits(a.m, a.n, a.k, compute_units));
    if (splits >= 1) {
        const int mt = wavek_row_blocks(a.m);
        const dim3 grid((unsigned)(a.n / 64), (unsigned)splits, (unsigned)((a.m + 16 * mt - 1) / (16 * mt)));
        float* part = (float*)workspace;
        switch (mt) {
        case 8: hipLaunchKernelGGL(wavek_linear_kernel<8>, grid, dim3(256), 0, stream, a, splits, part); break;
        case 4: hipLaunchKernelGGL(wavek_linear_kernel<4>, grid, dim3(256), 0, stream, a, splits, part); break;
        case 2: hipLaunchKernelGGL(wavek_linear_kernel<2>, grid, dim3(256), 0, stream, a, splits, part); break;
        default: hipLaunchKernelGGL(wavek_linear_kernel<1>, grid, dim3(256), 0, stream, a, splits, part); break;
        }
        reduce(splits);
        return kLaunchOk;
    }
    splits = fit(linear_splits(a.m, a.n, a.k, compute_units));
    if (splits >= 1) {
        hipLaunchKernelGGL(split_linear_kernel, dim3((unsigned)(a.n / kSplitCols), (unsigned)splits, (unsigned)mblocks),
                           dim3(kSplitThreads), 0, stream, a, splits, (float*)workspace);
        reduce(splits);
        return kLaunchOk;
    }
    hipLaunchKernelGGL(skinny_linear_kernel, dim3((unsigned)(a.n / kLinCols), (unsigned)mblocks), dim3(kLinThreads), 0, stream, a);
    return kLaunchOk;
}

} // namespace pmxhip
