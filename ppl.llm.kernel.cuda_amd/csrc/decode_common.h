// Device-side helpers shared by the decode attention kernels (included by their .hip files only).
#ifndef PMX_HIP_DECODE_COMMON_H_
#define PMX_HIP_DECODE_COMMON_H_

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
// STREAM adds the non-temporal hint.  Every cache byte is read once per step, and a plain read stream runs at
// 6.7 TB/s with the hint against 6.0 TB/s without it on this chip; but a hinted line does not stay in the
// cache for a second instruction, so the hint is for loads whose instruction covers whole 128-byte lines that
// nobody else reads: the int8 rows of the quad kernel (6 % faster; with its scale loads hinted too only 4 %),
// not the general kernel, whose lanes of a quad read different tokens (60 % slower with the hint).
template <bool STREAM>
__device__ __forceinline__ void load_b128(u32x4& dst, uint32_t lane_off, const char* wave_base)
{
    if (STREAM) asm volatile("global_load_dwordx4 %0, %1, %2 nt" : "=&v"(dst) : "v"(lane_off), "s"(wave_base) : "memory");
    else asm volatile("global_load_dwordx4 %0, %1, %2" : "=&v"(dst) : "v"(lane_off), "s"(wave_base) : "memory");
}
template <bool STREAM>
__device__ __forceinline__ void load_b32(uint32_t& dst, uint32_t lane_off, const char* wave_base)
{
    if (STREAM) asm volatile("global_load_dword %0, %1, %2 nt" : "=&v"(dst) : "v"(lane_off), "s"(wave_base) : "memory");
    else asm volatile("global_load_dword %0, %1, %2" : "=&v"(dst) : "v"(lane_off), "s"(wave_base) : "memory");
}
// waits until at most N vector memory operations are outstanding; the values pass through the
// statement so that no use of them can be scheduled before the wait
template <int N>
__device__ __forceinline__ void wait_loads(u32x4& a, uint32_t& b)
{
    asm volatile("s_waitcnt vmcnt(%2)" : "+v"(a), "+v"(b) : "n"(N));
}
template <int N>
__device__ __forceinline__ void wait_loads(uint32_t& a, uint32_t& b)
{
    asm volatile("s_waitcnt vmcnt(%2)" : "+v"(a), "+v"(b) : "n"(N));
}
// waits until at most N vector memory operations are outstanding, for a whole block's staging registers
template <int N>
__device__ __forceinline__ void wait_block(u32x4 (&q)[4], uint32_t (&sc)[4])
{
    asm volatile("s_waitcnt vmcnt(%8)"
                 : "+v"(q[0]), "+v"(q[1]), "+v"(q[2]), "+v"(q[3]), "+v"(sc[0]), "+v"(sc[1]), "+v"(sc[2]), "+v"(sc[3])
                 : "n"(N));
}
// one half (an attn_mask value) per lane, zero-extended
__device__ __forceinline__ void load_u16(uint32_t& dst, uint32_t lane_off, const char* wave_base)
{
    asm volatile("global_load_ushort %0, %1, %2" : "=&v"(dst) : "v"(lane_off), "s"(wave_base) : "memory");
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

// The ranges cut a stream in which every sequence is preceded by kSequenceCost positions that hold no token:
// a workgroup pays a fixed price for every sequence it starts (query rows, first cache block, merge and
// store of the piece), and with the price in the stream the ranges that start more sequences get fewer
// tokens.  Stream position of token t of sequence b: kvstarts[b] - kvstarts[0] + kSequenceCost * (b + 1) + t.
constexpr int kSequenceCost = 32; // measured: 32 to 64 serve ragged batches best (1.5-2 % over none)
__device__ __forceinline__ int64_t stream_length(int64_t tokens, int64_t sequences) { return tokens + kSequenceCost * sequences; }
__device__ __forceinline__ int64_t sequence_origin(int64_t first_token, int64_t b) { return first_token + kSequenceCost * (b + 1); }

// Tokens per range: equal shares rounded up to a whole number of workgroup
// iterations, never below kMinTokensPerRange.  Shared by both kernels.
__device__ __forceinline__ int64_t tokens_per_range(int64_t total, int ranges, int wg_tokens, int min_tokens)
{
    int64_t per = (total + ranges - 1) / ranges;
    if (per < min_tokens) per = min_tokens;
    return (per + wg_tokens - 1) / wg_tokens * wg_tokens;
}

// The piece [pa, pe) of a sequence (stream position s_beg, length len) that the range [r0, r1)
// owns, in sequence coordinates.  A cut inside the sequence moves up to the next multiple of
// `align` (a power of two) or to the sequence end; both neighbours compute the same cut, so the
// pieces of a sequence still partition it.  pe <= pa: the range owns nothing of the sequence.
__device__ __forceinline__ void piece_bounds(int64_t r0, int64_t r1, int64_t s_beg, int64_t len, int align,
                                             int64_t& pa, int64_t& pe)
{
    const int64_t mask = (int64_t)align - 1;
    int64_t lo = r0 - s_beg, hi = r1 - s_beg;
    lo = lo <= 0 ? 0 : ((lo + mask) & ~mask);
    hi = hi <= 0 ? 0 : ((hi + mask) & ~mask);
    pa = lo < len ? lo : len;
    pe = hi < len ? hi : len;
}

// first b in [0, n) whose stream interval ends beyond g: starts[b + 1] - starts[0] + kSequenceCost * (b + 1) > g
// (starts is non-decreasing).  Every workgroup runs this before it can request its first cache block, so the
// whole chip waits on it at the start of the kernel.  Up to kCountedSequences entries are counted by the lanes
// (the answer is the number of entries <= g): independent loads, one memory latency; beyond that, bisection
// with scalar loads (one latency per halving).
constexpr int kCountedSequences = 1024;
__device__ __forceinline__ int find_sequence(const_i64_ptr starts, const int64_t* starts_global, int n, int64_t g, int lane)
{
    const int64_t base = starts[0];
    if (n <= kCountedSequences) {
        int count = 0;
        for (int i0 = 0; i0 < n; i0 += kWave) {
            const int i = i0 + lane;
            const bool below = i < n && stream_length(starts_global[i + 1] - base, i + 1) <= g;
            count += __builtin_popcountll(__builtin_amdgcn_ballot_w64(below));
        }
        return count;
    }
    int lo = 0, hi = n; // answer in [lo, hi]
    while (lo < hi) {
        const int mid = (lo + hi) >> 1;
        if (stream_length(starts[mid + 1] - base, mid + 1) > g) hi = mid;
        else lo = mid + 1;
    }
    return lo;
}

// The same search, which also hands out starts[b] and starts[b + 1] of the sequence it finds (undefined when it
// returns n): in the counted form two lanes hold them already, so the workgroup's first piece does not begin with
// another pair of dependent loads.
__device__ __forceinline__ int64_t lane_value(int64_t v, int src_lane)
{
    const uint32_t lo = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)(uint64_t)v, src_lane);
    const uint32_t hi = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)((uint64_t)v >> 32), src_lane);
    return (int64_t)(((uint64_t)hi << 32) | lo);
}
__device__ __forceinline__ int find_sequence(const_i64_ptr starts, const int64_t* starts_global, int n, int64_t g, int lane,
                                             int64_t& seq_start, int64_t& seq_end)
{
    const int64_t base = starts[0];
    seq_start = base;
    seq_end = base;
    if (n <= kCountedSequences) {
        int count = 0;
        bool found = false;
        int64_t last_of_previous = base; // starts[i0] of the chunk in hand
        for (int i0 = 0; i0 < n; i0 += kWave) {
            const int i = i0 + lane;
            const int64_t end_i = i < n ? starts_global[i + 1] : base;
            const bool below = i < n && stream_length(end_i - base, i + 1) <= g;
            const int c = __builtin_popcountll(__builtin_amdgcn_ballot_w64(below)); // the lanes below come first
            count += c;
            if (!found && c < kWave) { // the sequence is entry i0 + c of this chunk (or there is none: i0 + c == n)
                found = true;
                seq_start = c > 0 ? lane_value(end_i, c - 1) : last_of_previous;
                seq_end = lane_value(end_i, c);
            }
            last_of_previous = lane_value(end_i, kWave - 1);
        }
        return count;
    }
    const int b = find_sequence(starts, starts_global, n, g, lane);
    if (b < n) {
        seq_start = starts[b];
        seq_end = starts[b + 1];
    }
    return b;
}


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

} // namespace
} // namespace pmxhip

#endif // PMX_HIP_DECODE_COMMON_H_
