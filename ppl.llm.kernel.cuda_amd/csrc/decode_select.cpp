// Which kernel runs the token ranges of a decode step, and the grouping of heads and tokens it implies.
// Host only.  The plan (pmxhip_decode_plan_make*) and the launch (pmxhip_decode_attention*) both come here, so
// the unit of the range cuts that the token-range kernel uses is by construction the one the combine kernel uses.
#include "launch_params.h"

namespace pmxhip {

namespace {

int largest_pow2_divisor_upto(int64_t n, int cap)
{
    int r = 1;
    while (r * 2 <= cap && n % (r * 2) == 0) r *= 2;
    return r;
}

// head_dim 64, 128 or 256: up to four query heads per kv head on one set of waves; head_dim 256, and head_dim 128
// with kv heads in eights: up to eight on two sets.  At head_dim 64 and 128 a wave holds two kv heads: an odd number of them leaves
// the last half-wave idle, which a single kv head does not pay for (half of every wave).
bool quad_serves(int64_t head_dim, int64_t g, int64_t num_kv_heads)
{
    if (head_dim == 256) return g <= 8;
    if ((head_dim != 128 && head_dim != 64) || num_kv_heads == 1) return false;
    return g <= 4 || (head_dim == 128 && g <= 8 && num_kv_heads % 8 == 0);
}

} // namespace

const char* decode_kernel_name(int32_t kernel)
{
    switch (kernel) {
        case kDecodeKernelGeneral: return "decode_attention_kernel";
        case kDecodeKernelQuad: return "decode_attention_quad_kernel";
        case kDecodeKernelMfma16: return "decode_attention_mfma16_kernel";
        case kDecodeKernelMfma32: return "decode_attention_mfma_kernel";
        default: return "";
    }
}

bool decode_choose(int64_t head_dim, int64_t num_heads, int64_t num_kv_heads, int32_t requested, DecodeChoice* out)
{
    if (head_dim != 64 && head_dim != 96 && head_dim != 128 && head_dim != 256) return false;
    if (num_kv_heads <= 0 || num_heads <= 0 || num_heads % num_kv_heads != 0) return false;
    const int64_t g = num_heads / num_kv_heads;
    int32_t kernel = requested;
    if (kernel == kDecodeKernelAuto) {
        // Many query heads per kv head: their VALU arithmetic outweighs the cache stream, so they become MFMA
        // columns (five and more; three and four as well on a single kv head, which would use half of the quad
        // kernel's lanes): 16 or 32 columns at head_dim 128, 32 at head_dim 64, and beyond 32 query heads per kv head
        // (multi-query models) as many passes of 32 columns as they need.  Up to four: the quad kernel, whose row
        // loads stream whole lines (head_dim 256: up to eight, on two sets of waves).  Everything else (head_dim 96,
        // a single kv head with one or two query heads, head_dim 256 with more than eight per kv head) stays on
        // the general kernel.
        if (head_dim == 128 && (g >= 5 || (g >= 3 && num_kv_heads == 1)))
            kernel = g <= kDecodeMfma16Columns ? kDecodeKernelMfma16 : kDecodeKernelMfma32;
        else if (head_dim == 64 && (g >= 5 || (g >= 3 && num_kv_heads == 1)))
            kernel = kDecodeKernelMfma32;
        else if (quad_serves(head_dim, g, num_kv_heads) && (g <= 4 || head_dim == 256))
            kernel = kDecodeKernelQuad;
        else
            kernel = kDecodeKernelGeneral;
    }
    DecodeChoice c{};
    c.kernel = kernel;
    switch (kernel) {
        case kDecodeKernelGeneral: {
            const int lanes_per_slot = head_dim == 64 ? 4 : (head_dim == 256 ? 16 : 8);
            const int slots_per_wave = 64 / lanes_per_slot;
            c.kv_heads_per_group = largest_pow2_divisor_upto(num_kv_heads, slots_per_wave < 8 ? slots_per_wave : 8);
            int gt = 1;
            while (gt < g && gt < 8) gt *= 2;
            c.q_heads_per_pass = gt;
            c.num_passes = (int32_t)((g + gt - 1) / gt);
            c.wg_tokens = decode_wg_tokens((int)head_dim, c.kv_heads_per_group);
            c.wgs_per_cu = 2;
            c.wgs_per_cu_short = c.wgs_per_cu;
            break;
        }
        case kDecodeKernelQuad: {
            if (!quad_serves(head_dim, g, num_kv_heads)) return false;
            // a wave holds two kv heads of 128 channels or one of 256; four, two or one waves per set
            const int per_wave = head_dim == 256 ? 1 : 2;
            const int64_t pairs = (num_kv_heads + per_wave - 1) / per_wave;
            c.kv_heads_per_group = per_wave * (pairs % 4 == 0 ? 4 : (pairs % 2 == 0 ? 2 : 1));
            c.q_heads_per_pass = g <= 1 ? 1 : (g <= 2 ? 2 : (g <= 4 ? 4 : 8)); // rows of the 4x4x4 products in use
            c.num_passes = 1;
            c.wg_tokens = head_dim == 64 ? 2 * kDecodeQuadTokens : kDecodeQuadTokens; // head_dim 64: blocks of 32 tokens
            // A CU holds eight of this kernel's waves, two per SIMD.  A long stream is cut for four, one per SIMD: the
            // second wave adds nothing to what the chip streams (each wave keeps three blocks of rows in flight), and
            // half as many ranges are half as many pieces to write and to combine.  Short batches, whose ranges are a
            // few blocks, still spread over all eight (their waves mostly wait), and so do the form with two sets of
            // waves per workgroup (head_dim 256 with more than four query heads per kv head: 43 against 57 us on 8 / 1
            // heads) and the workgroups of two waves (four kv heads: two such workgroups per CU ran 22 % slower than
            // four, 216 against 177 us -- their waves do not end up one per SIMD).
            const int waves = c.kv_heads_per_group / per_wave; // per set
            c.wgs_per_cu_short = 8 / waves;
            if (head_dim == 256 && g > 4) c.wgs_per_cu_short = c.wgs_per_cu_short > 1 ? c.wgs_per_cu_short / 2 : 1; // twice the waves per workgroup
            const bool one_per_simd = !(head_dim == 256 && g > 4) && waves != 2;
            c.wgs_per_cu = one_per_simd ? c.wgs_per_cu_short / 2 : c.wgs_per_cu_short;
            break;
        }
        case kDecodeKernelMfma16:
        case kDecodeKernelMfma32: {
            const int cols = kernel == kDecodeKernelMfma16 ? kDecodeMfma16Columns : kDecodeMfmaColumns;
            // the 16-column form: head_dim 128, one pass; the 32-column form: head_dim 128 or 64, any number of passes
            if (kernel == kDecodeKernelMfma16 ? (head_dim != 128 || g > cols) : (head_dim != 128 && head_dim != 64)) return false;
            c.kv_heads_per_group = num_kv_heads % 4 == 0 ? 4 : (num_kv_heads % 2 == 0 ? 2 : 1); // a wave per kv head
            c.q_heads_per_pass = cols;
            c.num_passes = (int32_t)((g + cols - 1) / cols);
            c.wg_tokens = kDecodeMfmaTokens;
            c.wgs_per_cu = kDecodeMfmaWavesPerCu / c.kv_heads_per_group;
            c.wgs_per_cu_short = c.wgs_per_cu;
            break;
        }
        default: return false;
    }
    *out = c;
    return true;
}

namespace {

// Bytes that the 32-bit lane offsets of a kernel span: the tokens of one wave block times the row stride, the kv
// heads that share a wave's 64-bit base times the head stride, and a row.
double lane_offset_span(const DecodeChoice& c, int64_t head_dim, int64_t stride_s, int64_t stride_h)
{
    int64_t tokens = c.wg_tokens, heads_apart = 0;
    switch (c.kernel) {
        case kDecodeKernelGeneral:
            tokens = c.wg_tokens / 4;               // a wave's block; the four waves have bases of their own
            heads_apart = c.kv_heads_per_group - 1; // every wave spans the group's kv heads
            break;
        case kDecodeKernelQuad:
            heads_apart = head_dim == 256 ? 0 : 1;  // the wave's second kv head; the first is in the wave's base
            break;
        default: break;                             // a wave per kv head: the head is in the base
    }
    return (double)tokens * (double)stride_s + (double)heads_apart * (double)stride_h + (double)head_dim;
}

} // namespace

bool decode_fit_cache_strides(int64_t head_dim, int64_t num_heads, int64_t num_kv_heads, int32_t requested,
                              int64_t stride_s, int64_t stride_h, DecodeChoice* c)
{
    constexpr double kLimit = 2147483648.0;
    if (stride_s < 0 || stride_h < 0) return false;
    if (lane_offset_span(*c, head_dim, stride_s, stride_h) < kLimit) return true;
    if (c->kernel == kDecodeKernelGeneral) {
        // fewer kv heads per wave (more tokens instead) until the heads' distance fits; one kv head per workgroup
        // has no head term at all
        while (c->kv_heads_per_group > 1) {
            c->kv_heads_per_group /= 2;
            c->wg_tokens = decode_wg_tokens((int)head_dim, c->kv_heads_per_group);
            if (lane_offset_span(*c, head_dim, stride_s, stride_h) < kLimit) return true;
        }
        return false;
    }
    if (c->kernel == kDecodeKernelQuad && requested == kDecodeKernelAuto) {
        // two kv heads further apart than a lane offset reaches: a kernel with a wave per kv head takes the step
        DecodeChoice alt;
        const int64_t g = num_heads / num_kv_heads;
        const int32_t other = head_dim == 128 && g <= kDecodeMfma16Columns ? kDecodeKernelMfma16
                              : (head_dim == 128 || head_dim == 64 ? kDecodeKernelMfma32 : kDecodeKernelGeneral);
        if (!decode_choose(head_dim, num_heads, num_kv_heads, other, &alt)) return false;
        *c = alt;
        return decode_fit_cache_strides(head_dim, num_heads, num_kv_heads, other, stride_s, stride_h, c);
    }
    return false;
}

bool decode_quad_launch_ok(const DecodeLaunch& a)
{
    if (a.output_stride_s % 8 != 0 || (reinterpret_cast<uintptr_t>(a.output) & 15u) != 0) return false;
    if (a.attn_mask != nullptr) {
        if (a.head_dim == 64) return false; // no mask form at head_dim 64
        if (a.num_kv_repeats > 4 || a.mask_stride_h < 0) return false;
        if (((double)a.num_heads * (double)a.mask_stride_h + 64.0) * 2.0 >= 4294967296.0) return false;
    }
    return true;
}

} // namespace pmxhip
