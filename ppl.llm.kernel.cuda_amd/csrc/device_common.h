// Device-side helpers shared by the gfx950 kernels of the int8-KV attention path.
#ifndef PMX_HIP_DEVICE_COMMON_H_
#define PMX_HIP_DEVICE_COMMON_H_

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace pmxhip {

typedef _Float16 half_t;
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int kWave = 64;
constexpr int kPage = 128; // tokens per page in cache_mode 1

template <typename T, typename U>
__device__ __forceinline__ T bitcast(const U& u)
{
    static_assert(sizeof(T) == sizeof(U), "bitcast size");
    return __builtin_bit_cast(T, u);
}

// ---- cross-lane exchange inside one 16-lane row (data-parallel primitives) ----
// XOR butterflies of width 1, 2, 4, 8 expressed as DPP controls: quad_perm for
// 1 and 2, row_half_mirror for 4 and row_mirror for 8 (valid once the narrower
// steps have made the value uniform inside each 4- resp. 8-lane group).
template <int CTRL>
__device__ __forceinline__ float dpp_f32(float v)
{
    return bitcast<float>(__builtin_amdgcn_update_dpp(0, bitcast<int>(v), CTRL, 0xf, 0xf, true));
}

constexpr int kDppXor1 = 0xB1;  // quad_perm:[1,0,3,2]
constexpr int kDppXor2 = 0x4E;  // quad_perm:[2,3,0,1]
constexpr int kDppHalfMirror = 0x141;
constexpr int kDppMirror = 0x140;

// Sum over the LANES-wide aligned lane group (LANES in {4, 8, 16}); every lane of
// the group ends with the total.
template <int LANES>
__device__ __forceinline__ float group_sum(float v)
{
    v += dpp_f32<kDppXor1>(v);
    v += dpp_f32<kDppXor2>(v);
    if (LANES >= 8) v += dpp_f32<kDppHalfMirror>(v);
    if (LANES >= 16) v += dpp_f32<kDppMirror>(v);
    return v;
}

// ---- int8 -> half ------------------------------------------------------------
// A byte b (two's complement x) with its top bit flipped is x + 128 as unsigned;
// under the exponent byte 0x64 the half 0x64uu equals 1024 + uu, so the half is
// 1152 + x exactly, and subtracting 1152 leaves x.  v_perm_b32 places bytes,
// one v_pk_add_f16 finishes two elements.
constexpr uint32_t kFlipSigns = 0x80808080u;
constexpr uint32_t kExpBytes = 0x64646464u;

__device__ __forceinline__ half2_t pk_sub_1152(uint32_t biased)
{
    const half2_t k = {(half_t)1152.0f, (half_t)1152.0f};
    return bitcast<half2_t>(biased) - k;
}

// bytes 0,1 of w (already sign-flipped) -> halves (x0, x1)
__device__ __forceinline__ half2_t cvt_bytes01(uint32_t flipped)
{
    return pk_sub_1152(__builtin_amdgcn_perm(kExpBytes, flipped, 0x04010400u));
}
__device__ __forceinline__ half2_t cvt_bytes23(uint32_t flipped)
{
    return pk_sub_1152(__builtin_amdgcn_perm(kExpBytes, flipped, 0x04030402u));
}

// byte K of two different words -> halves (a.byteK, b.byteK); inputs are raw
// (unflipped): the XOR supplies both the sign flip and the exponent byte.
template <int K>
__device__ __forceinline__ half2_t cvt_byte_pair(uint32_t a, uint32_t b)
{
    // selector bytes (LSB first): a.byteK, zero, b.byteK, zero; src0 = b (bytes 4-7), src1 = a
    constexpr uint32_t sel = (uint32_t)K | (0x0cu << 8) | ((uint32_t)(4 + K) << 16) | (0x0cu << 24);
    const uint32_t placed = __builtin_amdgcn_perm(b, a, sel);
    return pk_sub_1152(placed ^ 0x64806480u);
}

// signed byte K of a word -> fp32, one SDWA conversion (sign-extending byte select)
template <int K>
__device__ __forceinline__ float byte_to_f32(uint32_t w)
{
    float r;
    if (K == 0) asm("v_cvt_f32_i32_sdwa %0, sext(%1) dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:BYTE_0" : "=v"(r) : "v"(w));
    if (K == 1) asm("v_cvt_f32_i32_sdwa %0, sext(%1) dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:BYTE_1" : "=v"(r) : "v"(w));
    if (K == 2) asm("v_cvt_f32_i32_sdwa %0, sext(%1) dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:BYTE_2" : "=v"(r) : "v"(w));
    if (K == 3) asm("v_cvt_f32_i32_sdwa %0, sext(%1) dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:BYTE_3" : "=v"(r) : "v"(w));
    return r;
}

__device__ __forceinline__ float dot2(half2_t a, half2_t b, float c)
{
    return __builtin_amdgcn_fdot2(a, b, c, false);
}
// first link of a dot-product chain whose start value stays live: the three-address form writes a
// new register, where the accumulating two-address form would first need a copy of c
__device__ __forceinline__ float dot2_init(half2_t a, half2_t b, float c)
{
    float r;
    asm("v_dot2_f32_f16 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}

// max of three in one instruction.  Written as assembly because the compiler's fmaxf first passes every operand of
// unknown origin through a quieting v_max_f32 x, x (one more instruction per accumulator element); the operands
// here are products and sums of finite numbers or -inf, never a signalling NaN.
__device__ __forceinline__ float max3(float a, float b, float c)
{
    float r;
    asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}

// p - float(h.x) and p - float(h.y) in one instruction each: the mixed-precision fused multiply-add reads the
// half operand in place (exact: the conversion and the subtraction round once, and the result is representable
// whenever h is p rounded to half)
__device__ __forceinline__ float sub_half_lo(float p, half2_t h)
{
    float r;
    asm("v_fma_mix_f32 %0, %1, -1.0, %2 op_sel_hi:[1,0,0]" : "=v"(r) : "v"(h), "v"(p));
    return r;
}
__device__ __forceinline__ float sub_half_hi(float p, half2_t h)
{
    float r;
    asm("v_fma_mix_f32 %0, %1, -1.0, %2 op_sel:[1,0,0] op_sel_hi:[1,0,0]" : "=v"(r) : "v"(h), "v"(p));
    return r;
}

// Hand-off of wave-private LDS data between the lanes of one wave: stores by some lanes, then loads of the same
// bytes by others (or the reverse, before a tile is overwritten).  The wave's LDS operations execute in program
// order, so the hardware needs nothing; the wavefront-scope fence keeps the compiler from moving the accesses
// across this point (it emits no instruction), and the wave barrier keeps it from rescheduling around it.
__device__ __forceinline__ void wave_lds_handoff()
{
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
}

// Index arrays (kvstarts, cachestarts) are read-only for the whole launch and are read at
// wave-uniform addresses: viewing them through the constant address space lets the compiler use
// scalar loads (scalar cache, no vector registers, no vector wait count) for them.
typedef const int64_t __attribute__((address_space(4)))* const_i64_ptr;
__device__ __forceinline__ const_i64_ptr as_constant(const int64_t* p)
{
    return (const_i64_ptr)(uintptr_t)p;
}

// ---- token addressing ----------------------------------------------------------
// cache_mode 0: row = cachestarts[b] + t; cache_mode 1: row = table[t / 128] + t % 128.
template <bool PAGED>
__device__ __forceinline__ int64_t token_row(const int64_t* __restrict__ cachestarts, int64_t table_base, int64_t t)
{
    if (PAGED) return cachestarts[table_base + (t >> 7)] + (t & (kPage - 1));
    return cachestarts[table_base] + t;
}

} // namespace pmxhip

#endif // PMX_HIP_DEVICE_COMMON_H_
