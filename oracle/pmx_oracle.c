/*
 * TEST INFRASTRUCTURE ONLY -- CPU oracle for the int8-KV dynamic-batching path.
 *
 * This file restates, in plain C, the arithmetic of the reference's
 *   src/ppl/kernel/llm/cuda/pmx/multi_head_cache_attention/kernel.cu   (KC below)
 *   src/ppl/kernel/llm/cuda/pmx/multi_head_cache_attention/utils.cu    (UC below)
 *   src/ppl/kernel/llm/cuda/flash_attn2/src/mask.h                      (causal alignment)
 * so that the HIP kernels can be checked against it.  Nothing in the shipped
 * library links, loads or calls this file: only tests, the smoke check and the
 * cpu_baseline leg of the benchmark do.
 *
 * Pinning status of each function (what independent evidence fixes its result):
 *   pmx_oracle_kv_cache_quantize   pinned: hand-derived known answers, exhaustive
 *                                  fp16 sweep against an independent numpy
 *                                  restatement, invariants (tests/test_oracle_*).
 *                                  The reference holds no golden vectors for it.
 *   pmx_oracle_decode_attention    pinned: closed forms (kvlen=1, zero query,
 *                                  dominant key), torch SDPA on the dequantised
 *                                  cache, naive python loops on tiny inputs.
 *   pmx_oracle_prefill_attention   pinned: torch SDPA with explicit bottom-right
 *                                  causal mask, qlen=1 rows equal decode.
 *   pmx_oracle_prefill_attention_ex pinned: equals pmx_oracle_prefill_attention without the
 *                                  optional inputs; torch SDPA with an additive float mask
 *                                  (bias + alibi + causal) on the dequantised cache and on
 *                                  fp16 K/V.
 *   pmx_oracle_kv_cache_reorder    pinned: numpy gather + transpose of the same pages for a
 *                                  concrete pair of layouts; reorder followed by its inverse
 *                                  restores the pages and touches nothing else.
 *   pmx_oracle_rotary_position_embedding pinned: numpy complex multiplication by exp(i angle) in
 *                                  binary64 (half-ulp bound), position 0 = identity, pair norms
 *                                  preserved, linear scaling = rotation at pos / factor.  The
 *                                  reference's own bits (approximate __powf / __sincosf) are
 *                                  parity unpinned.
 *   pmx_oracle_splitkv_combine     pinned: any split of the kv range equals the
 *                                  single pass (log-sum-exp associativity).
 *   pmx_oracle_row_parallel_linear pinned: numpy matmul in binary64 of the same half inputs; exact
 *                                  small-integer products; identity weight = copy; bias alone for a
 *                                  zero input; linearity in the input.  The reference's own bits come
 *                                  from cublasLt (row_parallel_linear.cu:61-84, algorithm chosen at run
 *                                  time): parity unpinned at the bit level, inside the stated tolerance.
 *   The reference itself cannot be compiled here (CUDA, inline PTX, CUTLASS, and
 *   dependencies fetched at configure time), so bit patterns of its fp16
 *   attention output are "parity unpinned"; the contract is the fp32
 *   dequantised attention within 2e-3 abs / 1e-2 rel.
 *
 * All half-precision values travel as uint16_t bit patterns.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

/* ------------------------------------------------------------------------- */
/* IEEE binary16 <-> binary32, bit level, round-to-nearest-even, subnormals   */
/* kept (no flush-to-zero).                                                   */
/* ------------------------------------------------------------------------- */

static inline float bits_to_float(uint32_t u)
{
    float f;
    memcpy(&f, &u, 4);
    return f;
}

static inline uint32_t float_to_bits(float f)
{
    uint32_t u;
    memcpy(&u, &f, 4);
    return u;
}

float pmx_oracle_half_to_float(uint16_t h)
{
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    const uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    if (exp == 0) {
        if (man == 0)
            return bits_to_float(sign);
        /* subnormal: value = man * 2^-24, exactly representable in binary32 */
        float v = (float)man * (1.0f / 16777216.0f);
        return bits_to_float(float_to_bits(v) | sign);
    }
    if (exp == 31)
        return bits_to_float(sign | 0x7f800000u | (man << 13));
    return bits_to_float(sign | ((exp + 112u) << 23) | (man << 13));
}

uint16_t pmx_oracle_float_to_half(float f)
{
    const uint32_t x = float_to_bits(f);
    const uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
    const uint32_t ax = x & 0x7fffffffu;
    if (ax >= 0x7f800000u) /* inf / nan */
        return (uint16_t)(sign | 0x7c00u | ((ax > 0x7f800000u) ? 0x200u : 0u));
    if (ax >= 0x477ff000u) /* >= 65520 rounds to inf */
        return (uint16_t)(sign | 0x7c00u);
    if (ax < 0x33000001u) /* <= 2^-25 rounds to zero (tie at 2^-25 goes to even = 0) */
        return sign;
    int32_t e = (int32_t)(ax >> 23) - 127; /* unbiased exponent */
    uint32_t m = (ax & 0x7fffffu) | 0x800000u; /* 24-bit significand */
    int shift; /* bits dropped from the 24-bit significand */
    uint32_t base;
    if (e < -14) { /* subnormal half: unit = 2^-24 */
        shift = 13 + (-14 - e);
        base = 0;
    } else {
        shift = 13;
        base = (uint32_t)(e + 15) << 10;
    }
    uint32_t q = m >> shift;
    const uint32_t rem = m & ((1u << shift) - 1u);
    const uint32_t half_ulp = 1u << (shift - 1);
    if (rem > half_ulp || (rem == half_ulp && (q & 1u)))
        q += 1; /* may carry into the exponent field, which is the right result */
    if (e >= -14)
        q -= 0x400u; /* drop the implicit bit: base already holds the exponent */
    return (uint16_t)(sign | (base + q));
}

/* ------------------------------------------------------------------------- */
/* Token addressing shared by every stage.  KC:97-100 (store), KC:365-368     */
/* (decode), flash_fwd_kernel.h:621-632 (prefill: table entries are token      */
/* offsets, multiplied by the token stride).                                   */
/* ------------------------------------------------------------------------- */

static inline int64_t cache_token_index(const int64_t* cachestarts, int64_t cachestarts_stride_b,
                                        int64_t batch_id, int64_t pos, int32_t page_size)
{
    if (page_size <= 0)
        return cachestarts[batch_id] + pos;
    return cachestarts[batch_id * cachestarts_stride_b + pos / page_size] + pos % page_size;
}

/* ------------------------------------------------------------------------- */
/* Quantise/append.  KC:86-157 (kernel), KC:2013-2057 (launch).                */
/*   absmax in half (KC:133-137), scale = half(float(absmax)/127) (KC:139),    */
/*   clamp to eps = half(1e-5f) (KC:129,141-142), q = rint_even(half(x/scale)) */
/*   (KC:146), 8 channels per group, scale index = element index / 8           */
/*   (KC:125-126).  The half division is the correctly rounded quotient.       */
/* ------------------------------------------------------------------------- */

void pmx_oracle_quantize_group8(const uint16_t* x, int8_t* q, uint16_t* scale_out)
{
    const uint16_t eps_bits = pmx_oracle_float_to_half(1e-5f); /* 0x00A8 */
    const float eps = pmx_oracle_half_to_float(eps_bits);
    float amax = 0.0f;
    for (int i = 0; i < 8; ++i) {
        const float a = fabsf(pmx_oracle_half_to_float(x[i]));
        amax = amax > a ? amax : a; /* same select form as KC:135 */
    }
    uint16_t s_bits = pmx_oracle_float_to_half(amax / 127.0f);
    float s = pmx_oracle_half_to_float(s_bits);
    if (!(s > eps)) {
        s = eps;
        s_bits = eps_bits;
    }
    for (int i = 0; i < 8; ++i) {
        /* half / half: exact quotient rounded once to binary16.  Going through a
         * correctly rounded binary32 quotient is equivalent (24 >= 2*11+2). */
        const float quo = pmx_oracle_half_to_float(x[i]) / s;
        const float quo_h = pmx_oracle_half_to_float(pmx_oracle_float_to_half(quo));
        q[i] = (int8_t)(int)nearbyintf(quo_h); /* default mode: ties to even */
    }
    *scale_out = s_bits;
}

int pmx_oracle_kv_cache_quantize(
    const uint16_t* current_key, const uint16_t* current_value,
    const int64_t* seqstarts, const int64_t* cachestarts, const int64_t* start_pos,
    int64_t batch, int64_t layer_idx, int64_t num_kv_heads, int64_t head_dim,
    int32_t page_size, /* 0 = contiguous (cache_mode 0), 128 = paged (cache_mode 1) */
    int64_t current_key_stride_s, int64_t current_value_stride_s,
    int64_t cache_stride_s, int64_t cache_stride_l, int64_t cache_stride_h, int64_t cache_stride_kv,
    int64_t cachestarts_stride_b,
    int8_t* cache, uint16_t* scale)
{
    if (head_dim % 8 != 0)
        return 2;
    for (int64_t b = 0; b < batch; ++b) {
        const int64_t seqlen = seqstarts[b + 1] - seqstarts[b];
#pragma omp parallel for schedule(static)
        for (int64_t i = 0; i < seqlen; ++i) {
            const int64_t tok = cache_token_index(cachestarts, cachestarts_stride_b, b, start_pos[b] + i, page_size);
            const int64_t in_tok = seqstarts[b] + i;
            for (int64_t h = 0; h < num_kv_heads; ++h) {
                for (int64_t d0 = 0; d0 < head_dim; d0 += 8) {
                    const int64_t in_idx = h * head_dim + d0;
                    const int64_t k_out = tok * cache_stride_s + layer_idx * cache_stride_l + h * cache_stride_h + d0;
                    const int64_t v_out = k_out + cache_stride_kv;
                    pmx_oracle_quantize_group8(current_key + in_tok * current_key_stride_s + in_idx,
                                               cache + k_out, scale + k_out / 8);
                    pmx_oracle_quantize_group8(current_value + in_tok * current_value_stride_s + in_idx,
                                               cache + v_out, scale + v_out / 8);
                }
            }
        }
    }
    return 0;
}

/* ------------------------------------------------------------------------- */
/* Attention over the dequantised cache.                                       */
/*   dequant: float(int8) * float(scale) -- exact in binary32.  (KC:404,509    */
/*   round this product to half; the contract here is the unrounded product.)  */
/*   logit = attn_scale * dot(q, k^) (+ mask)  KC:410-415                      */
/*   kv head = q head / num_kv_repeats          KC:299                          */
/*   kv length = kvstarts[b+1]-kvstarts[b]      KC:347                          */
/*   softmax and PV accumulate in double; result written as binary32.          */
/* ------------------------------------------------------------------------- */

static void attend_one_row(
    const uint16_t* q_row, /* head_dim halves */
    const uint16_t* mask_row, /* may be NULL; indexed by kv position */
    const int8_t* cache, const uint16_t* scale,
    const int64_t* cachestarts, int64_t cachestarts_stride_b, int64_t b, int32_t page_size,
    int64_t kv_begin, int64_t kv_end, /* positions attended: [kv_begin, kv_end) */
    int64_t head_base, /* layer_idx*stride_l + kvh*stride_h */
    int64_t cache_stride_s, int64_t cache_stride_kv, int64_t head_dim, float attn_scale,
    double* logits, /* scratch, >= kv_end-kv_begin */
    float* out, /* head_dim floats */
    float* out_max, float* out_sum) /* optional: running max and exp-sum (for split tests) */
{
    float qf[256];
    for (int64_t d = 0; d < head_dim; ++d)
        qf[d] = pmx_oracle_half_to_float(q_row[d]);
    const int64_t n = kv_end - kv_begin;
    double mx = -INFINITY;
    for (int64_t t = 0; t < n; ++t) {
        const int64_t tok = cache_token_index(cachestarts, cachestarts_stride_b, b, kv_begin + t, page_size);
        const int64_t k_off = tok * cache_stride_s + head_base;
        double acc = 0.0;
        for (int64_t d0 = 0; d0 < head_dim; d0 += 8) {
            const float s = pmx_oracle_half_to_float(scale[(k_off + d0) >> 3]);
            for (int64_t d = d0; d < d0 + 8; ++d)
                acc += (double)qf[d] * (double)((float)cache[k_off + d] * s);
        }
        double l = (double)attn_scale * acc;
        if (mask_row)
            l += (double)pmx_oracle_half_to_float(mask_row[kv_begin + t]);
        logits[t] = l;
        if (l > mx)
            mx = l;
    }
    double o[256];
    for (int64_t d = 0; d < head_dim; ++d)
        o[d] = 0.0;
    double sum = 0.0;
    for (int64_t t = 0; t < n; ++t) {
        const double p = (mx == -INFINITY) ? 0.0 : exp(logits[t] - mx);
        sum += p;
        const int64_t tok = cache_token_index(cachestarts, cachestarts_stride_b, b, kv_begin + t, page_size);
        const int64_t v_off = tok * cache_stride_s + head_base + cache_stride_kv;
        for (int64_t d0 = 0; d0 < head_dim; d0 += 8) {
            const float s = pmx_oracle_half_to_float(scale[(v_off + d0) >> 3]);
            for (int64_t d = d0; d < d0 + 8; ++d)
                o[d] += p * (double)((float)cache[v_off + d] * s);
        }
    }
    const double inv = sum > 0.0 ? 1.0 / sum : 0.0;
    for (int64_t d = 0; d < head_dim; ++d)
        out[d] = (float)(o[d] * inv);
    if (out_max)
        *out_max = (float)mx;
    if (out_sum)
        *out_sum = (float)sum;
}

/* Decode: sequences [0, decoding_batches), one query row each, row index = batch
 * index (KC:333), output row likewise (KC:589).  Mask row for sequence b starts at
 * attn_mask + h*mask_stride_h + b*mask_stride_s + kvstarts[b] (KC:320-324). */
int pmx_oracle_decode_attention(
    const uint16_t* query, const uint16_t* attn_mask, /* mask may be NULL */
    const int8_t* cache, const uint16_t* scale,
    const int64_t* cachestarts, const int64_t* kvstarts,
    int64_t decoding_batches, int64_t num_heads, int64_t num_kv_heads, int64_t head_dim,
    float attn_scale, int64_t layer_idx, int32_t page_size,
    int64_t query_stride_s, int64_t output_stride_s, int64_t mask_stride_s, int64_t mask_stride_h,
    int64_t cache_stride_s, int64_t cache_stride_l, int64_t cache_stride_h, int64_t cache_stride_kv,
    int64_t cachestarts_stride_b,
    float* output) /* [decoding_batches, output_stride_s] binary32 */
{
    if (num_kv_heads <= 0 || num_heads % num_kv_heads != 0 || head_dim % 8 != 0 || head_dim > 256)
        return 2;
    const int64_t repeats = num_heads / num_kv_heads;
    int64_t max_len = 0;
    for (int64_t b = 0; b < decoding_batches; ++b) {
        const int64_t l = kvstarts[b + 1] - kvstarts[b];
        if (l > max_len)
            max_len = l;
    }
    const int64_t work = decoding_batches * num_heads;
#pragma omp parallel
    {
        double* logits = (double*)malloc(sizeof(double) * (size_t)(max_len > 0 ? max_len : 1));
#pragma omp for schedule(dynamic, 1)
        for (int64_t w = 0; w < work; ++w) {
            const int64_t b = w / num_heads, h = w % num_heads;
            const int64_t kvh = h / repeats;
            const int64_t len = kvstarts[b + 1] - kvstarts[b];
            const uint16_t* mrow = attn_mask ? attn_mask + h * mask_stride_h + b * mask_stride_s + kvstarts[b] : NULL;
            attend_one_row(query + b * query_stride_s + h * head_dim, mrow, cache, scale,
                           cachestarts, cachestarts_stride_b, b, page_size, 0, len,
                           layer_idx * cache_stride_l + kvh * cache_stride_h,
                           cache_stride_s, cache_stride_kv, head_dim, attn_scale, logits,
                           output + b * output_stride_s + h * head_dim, NULL, NULL);
        }
        free(logits);
    }
    return 0;
}

/* Prefill over the int8 cache: sequences [decoding_batches, batch).  Query rows
 * seqstarts[b]..seqstarts[b+1] (KC:2131), kv length from kvstarts (KC:2132),
 * cache rows through cachestarts (KC:2142).  Causal mask is bottom-right aligned:
 * row i sees columns < i + 1 + kvlen - qlen (flash_attn2/src/mask.h:186). */
int pmx_oracle_prefill_attention(
    const uint16_t* query,
    const int8_t* cache, const uint16_t* scale,
    const int64_t* seqstarts, const int64_t* kvstarts, const int64_t* cachestarts,
    int64_t batch, int64_t decoding_batches, int32_t is_causal,
    int64_t num_heads, int64_t num_kv_heads, int64_t head_dim,
    float attn_scale, int64_t layer_idx, int32_t page_size,
    int64_t query_stride_s, int64_t output_stride_s,
    int64_t cache_stride_s, int64_t cache_stride_l, int64_t cache_stride_h, int64_t cache_stride_kv,
    int64_t cachestarts_stride_b,
    float* output) /* indexed by absolute query row like the query */
{
    if (num_kv_heads <= 0 || num_heads % num_kv_heads != 0 || head_dim % 8 != 0 || head_dim > 256)
        return 2;
    const int64_t repeats = num_heads / num_kv_heads;
    for (int64_t b = decoding_batches; b < batch; ++b) {
        const int64_t qlen = seqstarts[b + 1] - seqstarts[b];
        const int64_t kvlen = kvstarts[b + 1] - kvstarts[b];
        const int64_t work = qlen * num_heads;
#pragma omp parallel
        {
            double* logits = (double*)malloc(sizeof(double) * (size_t)(kvlen > 0 ? kvlen : 1));
#pragma omp for schedule(dynamic, 8)
            for (int64_t w = 0; w < work; ++w) {
                const int64_t i = w / num_heads, h = w % num_heads;
                const int64_t kvh = h / repeats;
                int64_t limit = kvlen;
                if (is_causal) {
                    limit = i + 1 + kvlen - qlen;
                    if (limit > kvlen)
                        limit = kvlen;
                    if (limit < 0)
                        limit = 0;
                }
                const int64_t row = seqstarts[b] + i;
                attend_one_row(query + row * query_stride_s + h * head_dim, NULL, cache, scale,
                               cachestarts, cachestarts_stride_b, b, page_size, 0, limit,
                               layer_idx * cache_stride_l + kvh * cache_stride_h,
                               cache_stride_s, cache_stride_kv, head_dim, attn_scale, logits,
                               output + row * output_stride_s + h * head_dim, NULL, NULL);
            }
            free(logits);
        }
    }
    return 0;
}

/* Prefill with every optional input of the two flash_attn2 calls of forward_prefill
 * (KC:2134-2212):
 *   - K/V either from the int8 cache (enable_cache_prefill, KC:2134-2179) or, with
 *     current_key != NULL, from the step's own fp16 current_key/current_value rows with
 *     kv length = query length (seqstart_k = seqstart_q, KC:2181-2212);
 *   - attn_mask: additive fp16 bias, block-diagonal over the batch: element (head h, absolute
 *     query row r, absolute kv column c) at h*mask_stride_h + r*mask_stride_s + c, added to the
 *     scaled logit (flash_attn2/src/flash_api.cu:171 scales it by 1/attn_scale before the
 *     softmax scale is applied; block_info.h:48-58 gives the offsets);
 *   - alibi_slopes: float32 per head; causal: + slope * col, otherwise
 *     - slope * |row + kvlen - qlen - col| (flash_attn2/src/mask.h:191-197, slope divided by
 *     the softmax scale at flash_fwd_kernel.h:764, i.e. applied to the scaled logit).
 * kv columns are absolute positions in the kv stream: kvstarts[b] + t for the cache path,
 * seqstarts[b] + t for the current_key path. */
int pmx_oracle_prefill_attention_ex(
    const uint16_t* query,
    const int8_t* cache, const uint16_t* scale,
    const uint16_t* current_key, const uint16_t* current_value, int64_t key_stride_s, int64_t value_stride_s,
    const uint16_t* attn_mask, int64_t mask_stride_s, int64_t mask_stride_h,
    const float* alibi_slopes,
    const int64_t* seqstarts, const int64_t* kvstarts, const int64_t* cachestarts,
    int64_t batch, int64_t decoding_batches, int32_t is_causal,
    int64_t num_heads, int64_t num_kv_heads, int64_t head_dim,
    float attn_scale, int64_t layer_idx, int32_t page_size,
    int64_t query_stride_s, int64_t output_stride_s,
    int64_t cache_stride_s, int64_t cache_stride_l, int64_t cache_stride_h, int64_t cache_stride_kv,
    int64_t cachestarts_stride_b,
    float* output)
{
    if (num_kv_heads <= 0 || num_heads % num_kv_heads != 0 || head_dim % 8 != 0 || head_dim > 256)
        return 2;
    const int64_t repeats = num_heads / num_kv_heads;
    const int from_current = current_key != NULL;
    for (int64_t b = decoding_batches; b < batch; ++b) {
        const int64_t qlen = seqstarts[b + 1] - seqstarts[b];
        const int64_t kvlen = from_current ? qlen : kvstarts[b + 1] - kvstarts[b];
        const int64_t col0 = from_current ? seqstarts[b] : kvstarts[b];
        const int64_t work = qlen * num_heads;
#pragma omp parallel
        {
            double* logits = (double*)malloc(sizeof(double) * (size_t)(kvlen > 0 ? kvlen : 1));
            float* kv = (float*)malloc(sizeof(float) * (size_t)head_dim);
#pragma omp for schedule(dynamic, 8)
            for (int64_t w = 0; w < work; ++w) {
                const int64_t i = w / num_heads, h = w % num_heads;
                const int64_t kvh = h / repeats;
                int64_t limit = kvlen;
                if (is_causal) {
                    limit = i + 1 + kvlen - qlen;
                    if (limit > kvlen) limit = kvlen;
                    if (limit < 0) limit = 0;
                }
                const int64_t row = seqstarts[b] + i;
                const uint16_t* q_row = query + row * query_stride_s + h * head_dim;
                double mx = -INFINITY;
                for (int64_t t = 0; t < limit; ++t) {
                    double acc = 0.0;
                    if (from_current) {
                        const uint16_t* k = current_key + (seqstarts[b] + t) * key_stride_s + kvh * head_dim;
                        for (int64_t d = 0; d < head_dim; ++d)
                            acc += (double)pmx_oracle_half_to_float(q_row[d]) * (double)pmx_oracle_half_to_float(k[d]);
                    } else {
                        const int64_t tok = cache_token_index(cachestarts, cachestarts_stride_b, b, t, page_size);
                        const int64_t k_off = tok * cache_stride_s + layer_idx * cache_stride_l + kvh * cache_stride_h;
                        for (int64_t d0 = 0; d0 < head_dim; d0 += 8) {
                            const float sc = pmx_oracle_half_to_float(scale[(k_off + d0) >> 3]);
                            for (int64_t d = d0; d < d0 + 8; ++d)
                                acc += (double)pmx_oracle_half_to_float(q_row[d]) * (double)((float)cache[k_off + d] * sc);
                        }
                    }
                    double l = (double)attn_scale * acc;
                    if (attn_mask)
                        l += (double)pmx_oracle_half_to_float(attn_mask[h * mask_stride_h + row * mask_stride_s + col0 + t]);
                    if (alibi_slopes) {
                        if (is_causal)
                            l += (double)alibi_slopes[h] * (double)t;
                        else
                            l -= (double)alibi_slopes[h] * fabs((double)(i + kvlen - qlen - t));
                    }
                    logits[t] = l;
                    if (l > mx) mx = l;
                }
                double o[256];
                for (int64_t d = 0; d < head_dim; ++d) o[d] = 0.0;
                double sum = 0.0;
                for (int64_t t = 0; t < limit; ++t) {
                    const double p = (mx == -INFINITY) ? 0.0 : exp(logits[t] - mx);
                    sum += p;
                    if (from_current) {
                        const uint16_t* v = current_value + (seqstarts[b] + t) * value_stride_s + kvh * head_dim;
                        for (int64_t d = 0; d < head_dim; ++d) o[d] += p * (double)pmx_oracle_half_to_float(v[d]);
                    } else {
                        const int64_t tok = cache_token_index(cachestarts, cachestarts_stride_b, b, t, page_size);
                        const int64_t v_off = tok * cache_stride_s + layer_idx * cache_stride_l + kvh * cache_stride_h + cache_stride_kv;
                        for (int64_t d0 = 0; d0 < head_dim; d0 += 8) {
                            const float sc = pmx_oracle_half_to_float(scale[(v_off + d0) >> 3]);
                            for (int64_t d = d0; d < d0 + 8; ++d) o[d] += p * (double)((float)cache[v_off + d] * sc);
                        }
                    }
                }
                const double inv = sum > 0.0 ? 1.0 / sum : 0.0;
                float* out = output + row * output_stride_s + h * head_dim;
                for (int64_t d = 0; d < head_dim; ++d) out[d] = (float)(o[d] * inv);
            }
            free(kv);
            free(logits);
        }
    }
    return 0;
}

/* One piece of one sequence: attention over kv positions [kv_begin, kv_end) of
 * sequence b for query head h, returning the normalised partial output plus the
 * piece's running max and exp-sum.  Used to check split-KV partials. */
int pmx_oracle_decode_partial(
    const uint16_t* query, const int8_t* cache, const uint16_t* scale,
    const int64_t* cachestarts,
    int64_t b, int64_t h, int64_t kv_begin, int64_t kv_end,
    int64_t num_heads, int64_t num_kv_heads, int64_t head_dim,
    float attn_scale, int64_t layer_idx, int32_t page_size,
    int64_t query_stride_s,
    int64_t cache_stride_s, int64_t cache_stride_l, int64_t cache_stride_h, int64_t cache_stride_kv,
    int64_t cachestarts_stride_b,
    float* out, float* out_max, float* out_sum)
{
    const int64_t repeats = num_heads / num_kv_heads;
    const int64_t n = kv_end - kv_begin;
    double* logits = (double*)malloc(sizeof(double) * (size_t)(n > 0 ? n : 1));
    attend_one_row(query + b * query_stride_s + h * head_dim, NULL, cache, scale,
                   cachestarts, cachestarts_stride_b, b, page_size, kv_begin, kv_end,
                   layer_idx * cache_stride_l + (h / repeats) * cache_stride_h,
                   cache_stride_s, cache_stride_kv, head_dim, attn_scale, logits,
                   out, out_max, out_sum);
    free(logits);
    return 0;
}

/* Split-KV combine.  KC:617-665: weights exp(lse_i - max lse) / sum, with
 * lse_i = m_i + log(l_i) (KC:450).  Here each piece carries (m_i, l_i) and a
 * normalised partial o_i; an empty piece has l_i = 0 and contributes nothing. */
int pmx_oracle_splitkv_combine(
    const float* partial_out, /* [n_pieces, head_dim] */
    const float* partial_max, const float* partial_sum, /* [n_pieces] */
    int64_t n_pieces, int64_t head_dim,
    float* out) /* [head_dim] */
{
    double mx = -INFINITY;
    for (int64_t i = 0; i < n_pieces; ++i)
        if (partial_sum[i] > 0.0f && (double)partial_max[i] > mx)
            mx = (double)partial_max[i];
    double den = 0.0;
    double o[256];
    for (int64_t d = 0; d < head_dim; ++d)
        o[d] = 0.0;
    for (int64_t i = 0; i < n_pieces; ++i) {
        if (!(partial_sum[i] > 0.0f))
            continue;
        const double w = (double)partial_sum[i] * exp((double)partial_max[i] - mx);
        den += w;
        for (int64_t d = 0; d < head_dim; ++d)
            o[d] += w * (double)partial_out[i * head_dim + d];
    }
    for (int64_t d = 0; d < head_dim; ++d)
        out[d] = den > 0.0 ? (float)(o[d] / den) : 0.0f;
    return 0;
}

/* Quotient identity that a quantiser may use instead of one division per channel (not from the
 * reference; a property of the arithmetic above that tests check): with rcp = 1.0f / s,
 * q0 = x * rcp, e = fmaf(-q0, s, x), quo = fmaf(e, rcp, q0), the int8 result
 * rint_even(half(quo)) equals rint_even(half(x / s)).  Compared here for EVERY finite half x and
 * every half scale s >= eps (2.0e9 pairs); returns the number of pairs whose int8 results differ
 * and, through *half_differs, the number whose half quotients differ in bits (-0 / s gives +0). */
int64_t pmx_oracle_count_reciprocal_quotient_mismatches(int64_t* half_differs)
{
    const int eps_bits = pmx_oracle_float_to_half(1e-5f);
    int64_t bad_q = 0, bad_h = 0;
#pragma omp parallel for reduction(+ : bad_q, bad_h) schedule(dynamic, 64)
    for (int sb = eps_bits; sb < 0x7C00; ++sb) {
        const float s = pmx_oracle_half_to_float((uint16_t)sb);
        const float rcp = 1.0f / s;
        for (int xb = 0; xb < 0x10000; ++xb) {
            if ((xb & 0x7C00) == 0x7C00) continue; /* inf, nan */
            const float x = pmx_oracle_half_to_float((uint16_t)xb);
            const uint16_t a = pmx_oracle_float_to_half(x / s);
            const float q0 = x * rcp;
            const uint16_t b = pmx_oracle_float_to_half(fmaf(fmaf(-q0, s, x), rcp, q0));
            if (a == b) continue;
            ++bad_h;
            const float fa = pmx_oracle_half_to_float(a), fb = pmx_oracle_half_to_float(b);
            if (fabsf(fa) < 1e9f && fabsf(fb) < 1e9f && (int)nearbyintf(fa) == (int)nearbyintf(fb)) continue;
            ++bad_q;
        }
    }
    if (half_differs) *half_differs = bad_h;
    return bad_q;
}

/* Host threads the OpenMP loops above will use (reported beside CPU timings). */
int pmx_oracle_num_threads(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* ------------------------------------------------------------------------- */
/* kv_cache_reorder / kv_cache_invert_reorder (pmx/kv_cache_reorder.cu:24-65,   */
/* 103-144): one byte per (slot, layer, plane, head, token, d), index formulas */
/* as in the reference, including head_dim as the tokens of a page (line 44).  */
/* stride arrays: {p, l, kv, h, t, d} for the cache, then the same for scales. */
/* ------------------------------------------------------------------------- */
int pmx_oracle_kv_cache_reorder(
    int32_t invert,
    uint8_t* kv_cache, uint8_t* kv_scale, uint8_t* outer_mem, const int64_t* page_ids,
    const int32_t* src_stride, const int32_t* dst_stride,
    int64_t page_nums, int64_t layers, int64_t kv_heads, int64_t tokens, int64_t head_dim, int64_t group_size,
    int64_t tp_rank, int64_t tp_size)
{
    const int64_t pcb = src_stride[0], psb = src_stride[6];
    const int64_t scale_row = head_dim / group_size * 2;
    const int32_t* cs = invert ? dst_stride : src_stride; /* cache-side strides */
    const int32_t* os = invert ? src_stride : dst_stride; /* outer-side strides */
    for (int64_t j = 0; j < page_nums; ++j) {
        const int64_t page = page_ids[j];
        uint8_t* outer_cache = outer_mem + (pcb + psb) * tp_size * j + tp_rank * pcb;
        uint8_t* outer_scale = outer_cache + (tp_size - tp_rank) * pcb + tp_rank * psb;
        for (int64_t l = 0; l < layers; ++l)
            for (int64_t kv = 0; kv < 2; ++kv)
                for (int64_t h = 0; h < kv_heads; ++h)
                    for (int64_t t = 0; t < tokens; ++t)
                        for (int64_t d = 0; d < head_dim; ++d) {
                            const int64_t ci = page * head_dim * head_dim + l * cs[1] + kv * cs[2] + h * cs[3] + t * cs[4] + d * cs[5];
                            const int64_t oi = l * os[1] + kv * os[2] + h * os[3] + t * os[4] + d * os[5];
                            if (invert) kv_cache[ci] = outer_cache[oi];
                            else outer_cache[oi] = kv_cache[ci];
                            if (d < scale_row) {
                                const int64_t si = page * head_dim * scale_row + l * cs[7] + kv * cs[8] + h * cs[9] + t * cs[10] + d * cs[11];
                                const int64_t so = l * os[7] + kv * os[8] + h * os[9] + t * os[10] + d * os[11];
                                if (invert) kv_scale[si] = outer_scale[so];
                                else outer_scale[so] = kv_scale[si];
                            }
                        }
    }
    return 0;
}

/* ------------------------------------------------------------------------- */
/* Rotary position embedding for dynamic batches                              */
/* (pmx/rotary_position_embedding.cu:35-91 coefficients, 268-343 kernel).      */
/* Pairs (2i, 2i+1), i < rotary_dim/2: (x, y) -> (x c - y s, y c + x s) in      */
/* binary32, rounded to half; other channels copied.  The angle follows the    */
/* reference formula 1.0f / powf(theta, i / (rotary_dim/2)) * pos with pow, cos */
/* and sin evaluated in binary64 and rounded once (the reference uses the      */
/* approximate __powf / __sincosf, whose bits are unpinned).                    */
/* scaling_type: 0 none, 1 linear, 2 dynamic.                                   */
/* ------------------------------------------------------------------------- */
int pmx_oracle_rotary_position_embedding(
    const uint16_t* query, const uint16_t* key,
    const int64_t* start_pos, const int64_t* seqstarts,
    float theta, int32_t bypass_key, int64_t rotary_dim, int64_t batch,
    int64_t num_heads, int64_t num_key_heads, int64_t head_dim,
    int64_t max_position_embeddings, int32_t scaling_type, float scaling_factor,
    int64_t query_stride_s, int64_t key_stride_s, int64_t rotated_query_stride_s, int64_t rotated_key_stride_s,
    uint16_t* rotated_query, uint16_t* rotated_key)
{
    if (head_dim % 2 != 0 || rotary_dim % 2 != 0 || rotary_dim > head_dim || scaling_type < 0 || scaling_type > 2)
        return 4;
    const int64_t rd2 = rotary_dim / 2;
    for (int64_t b = 0; b < batch; ++b) {
        const int64_t seqlen = seqstarts[b + 1] - seqstarts[b];
        float th = theta;
        if (scaling_type == 2) {
            const int64_t pos_end = start_pos[b] + seqlen;
            if (pos_end > max_position_embeddings) {
                const float base = ((scaling_factor * (float)pos_end) / (float)max_position_embeddings) - (scaling_factor - 1.f);
                const float expn = (float)rd2 / (float)(rd2 - 1);
                th = theta * (float)pow((double)base, (double)expn);
            }
        }
        for (int64_t sidx = 0; sidx < seqlen; ++sidx) {
            const int64_t tok = seqstarts[b] + sidx;
            const int64_t pos = start_pos[b] + sidx;
            for (int64_t h = 0; h < num_heads; ++h)
                for (int64_t i = 0; i < head_dim / 2; ++i) {
                    float c = 1.f, sn = 0.f;
                    if (i < rd2) {
                        const float inv = 1.0f / (float)pow((double)th, (double)((float)i / (float)rd2));
                        const float p = scaling_type == 1 ? (float)pos / scaling_factor : (float)pos;
                        const float angle = inv * p;
                        c = (float)cos((double)angle);
                        sn = (float)sin((double)angle);
                    }
                    for (int which = 0; which < 2; ++which) {
                        if (which == 1 && h >= num_key_heads) continue;
                        const uint16_t* src = which == 0 ? query + tok * query_stride_s : key + tok * key_stride_s;
                        uint16_t* dst = which == 0 ? rotated_query + tok * rotated_query_stride_s : rotated_key + tok * rotated_key_stride_s;
                        const int64_t e = h * head_dim + 2 * i;
                        if (i >= rd2 || (which == 1 && bypass_key)) {
                            dst[e] = src[e];
                            dst[e + 1] = src[e + 1];
                        } else {
                            const float x = pmx_oracle_half_to_float(src[e]), y = pmx_oracle_half_to_float(src[e + 1]);
                            dst[e] = pmx_oracle_float_to_half(x * c - y * sn);
                            dst[e + 1] = pmx_oracle_float_to_half(y * c + x * sn);
                        }
                    }
                }
        }
    }
    return 0;
}

/* Single-rank row_parallel_linear (src/ppl/kernel/llm/cuda/pmx/row_parallel_linear.cu:25-110 with
 * nccl_param->size == 1): output(M, N) = input(M, K) * weight(N, K)^T + bias, half tensors; the reference's
 * cublasLt GEMM accumulates in float32 and rounds once to half (alpha 1, beta 0, bias as epilogue).  Here the
 * float32 sum runs over k in index order.  Strides in halves per row.  bias may be NULL. */
int pmx_oracle_row_parallel_linear(const uint16_t* input, const uint16_t* weight, const uint16_t* bias, int64_t m, int64_t n,
                                   int64_t k, int64_t input_stride, int64_t weight_stride, int64_t output_stride,
                                   uint16_t* output)
{
    if (m < 0 || n < 0 || k < 0 || !input || !weight || !output) return 1;
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < m; ++i) {
        for (int64_t j = 0; j < n; ++j) {
            const uint16_t* a = input + i * input_stride;
            const uint16_t* w = weight + j * weight_stride;
            float acc = 0.0f;
            for (int64_t c = 0; c < k; ++c) acc += pmx_oracle_half_to_float(a[c]) * pmx_oracle_half_to_float(w[c]);
            if (bias) acc += pmx_oracle_half_to_float(bias[j]);
            output[i * output_stride + j] = pmx_oracle_float_to_half(acc);
        }
    }
    return 0;
}
