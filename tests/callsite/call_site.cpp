// A stand-alone translation unit written the way a serving engine's op kernel calls the reference operator
// (include/ppl/kernel/llm/cuda/pmx/multi_head_cache_attention.h:107-158, kv_cache_reorder.h:42-74,
// rotary_position_embedding.h:54-76), against this library's headers: the include lines and the two HIP type
// names are the only differences from such a call site.  Compiled with a plain C++ compiler (no device code),
// linked with libpmx_hip.so and run on the host by tests/test_cpp_call_site.py: heuristic_prepare is pure host
// code, and the stage calls below are made on an empty batch, which returns before any launch.
#include <cinttypes>
#include <cstdio>

#include "pmx_hip/cache_attention.h"
#include "pmx_hip/key_value_cache.h"
#include "pmx_hip/kv_cache_reorder.h"
#include "pmx_hip/rotary_position_embedding.h"
#include "pmx_hip/row_parallel_linear.h"

namespace pmx = ppl::kernel::llm::cuda::pmx;

// the prototypes of the reference, spelled out: assigning the library's functions to them fails to compile if an
// argument was dropped, added or reordered
typedef ppl::common::RetCode (*reorder_fn)(hipStream_t, const void*, const void*, const void*, const pmx::Stride&,
                                           const pmx::Stride&, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t,
                                           int64_t, int64_t, void*);
typedef ppl::common::RetCode (*invert_reorder_fn)(hipStream_t, const void*, const void*, const pmx::Stride&,
                                                  const pmx::Stride&, int64_t, int64_t, int64_t, int64_t, int64_t,
                                                  int64_t, int64_t, int64_t, void*, void*);
typedef ppl::common::RetCode (*linear_fn)(const hipStream_t, const cublasLtHandle_t&, const cublasLtMatmulAlgo_t*,
                                          const ppl::common::TensorShape*, const void*, const ppl::common::TensorShape*,
                                          const void*, const ppl::common::TensorShape*, const void*, const int64_t, const int64_t,
                                          const ppl::common::NcclParam*, const bool, void*, const int64_t, void*,
                                          const ppl::common::TensorShape*, void*, const bool);
typedef ppl::common::RetCode (*rope_fn)(hipStream_t, const ppl::common::TensorShape*, const void*,
                                        const ppl::common::TensorShape*, const void*, const void*, const void*, const float,
                                        const int32_t, const int64_t, const int64_t, const int64_t, const int64_t,
                                        const int64_t, const int64_t, const pmx::rope_scaling_t, const float,
                                        const ppl::common::TensorShape*, void*, const ppl::common::TensorShape*, void*);

int main()
{
    // Llama-3-8B decode step: 128 sequences, 32 query / 8 kv heads of 128 channels, paged cache
    const int64_t batch = 128, decoding_batches = 128, num_heads = 32, num_kv_heads = 8, head_dim = 128;
    const int64_t max_seqlen = 1, max_kvlen = 8192, layer_idx = 3, num_layer = 32, pool_tokens = 1 << 20;
    hipDeviceProp_t device_prop = {};
    device_prop.multiProcessorCount = 256;
    device_prop.sharedMemPerBlockOptin = 160 * 1024;

    ppl::common::TensorShape query_shape(ppl::common::DATATYPE_FLOAT16, {batch, num_heads, head_dim});
    ppl::common::TensorShape key_shape(ppl::common::DATATYPE_FLOAT16, {batch, num_kv_heads, head_dim});
    ppl::common::TensorShape mask_shape;
    // device pointers are only stored by heuristic_prepare; any non-null values serve on the host
    void* const query = (void*)0x10000;
    void* const current_key = (void*)0x20000;
    void* const current_value = (void*)0x30000;
    void* const seqstarts = (void*)0x40000;
    void* const kvstarts = (void*)0x50000;
    void* const cachestarts = (void*)0x60000;
    void* const start_pos = (void*)0x70000;
    void* const cache = (void*)0x100000;
    void* const scale = (void*)0x200000;
    void* const output = (void*)0x80000;
    const int64_t cache_stride_s = num_kv_heads * head_dim, cache_stride_h = head_dim;
    const int64_t cache_stride_kv = pool_tokens * cache_stride_s, cache_stride_l = 2 * cache_stride_kv;

    pmx::dynamic_batching_multi_head_cache_attention attn;
    ppl::common::RetCode rc = attn.heuristic_prepare(
        device_prop,
        &query_shape, query,
        &key_shape, current_key,
        &key_shape, current_value,
        &mask_shape, nullptr,
        seqstarts, kvstarts, cachestarts, start_pos,
        nullptr, // alibi_slopes
        true,    // is_causal
        batch, decoding_batches, max_seqlen, max_kvlen,
        layer_idx, num_layer, num_heads, num_kv_heads, head_dim,
        1, 128, // cache_mode, page_size
        cache_stride_s, cache_stride_l, cache_stride_h, cache_stride_kv,
        64,   // cachestarts_stride_b
        true, // enable_cache_prefill
        true, true, true, // enable_sharemem_mhca, enable_infinity_mhca, enable_infinity_gqca
        1, 0, // specify_decoding_multi_block, specify_decoding_tpb
        cache, scale,
        &query_shape, output);
    printf("prepare rc=%u\n", (unsigned)rc);
    const auto& cfg = attn.cfg;
    printf("prefill_batches=%" PRId64 " q_stride_s=%" PRId64 " k_stride_s=%" PRId64 " o_stride_s=%" PRId64
           " num_kv_repeats=%" PRId64 " attn_scale=%.9g decoding_algo=%d multi_block=%" PRId64 " workspace_size=%" PRId64 "\n",
           cfg.prefill_batches, cfg.q_stride_s, cfg.k_stride_s, cfg.o_stride_s, cfg.num_kv_repeats, (double)cfg.attn_scale,
           (int)cfg.decoding_algo, cfg.decoding_multi_block_size, cfg.workspace_size);
    printf("device_prop kept by pointer: %d\n", (int)(cfg.device_prop == &device_prop));
    attn.cfg.workspace = (void*)0x300000; // the caller's job after heuristic_prepare (reference header, lines 104-106)

    // a rejected configuration: 30 query heads over 8 kv heads (utils.cu:101-105)
    ppl::common::TensorShape bad_shape(ppl::common::DATATYPE_FLOAT16, {batch, 30, head_dim});
    pmx::dynamic_batching_multi_head_cache_attention bad;
    rc = bad.heuristic_prepare(device_prop, &bad_shape, query, &key_shape, current_key, &key_shape, current_value, &mask_shape,
                               nullptr, seqstarts, kvstarts, cachestarts, start_pos, nullptr, true, batch, decoding_batches,
                               max_seqlen, max_kvlen, layer_idx, num_layer, 30, num_kv_heads, head_dim, 1, 128, cache_stride_s,
                               cache_stride_l, cache_stride_h, cache_stride_kv, 64, true, true, true, true, 1, 0, cache, scale,
                               &bad_shape, output);
    printf("bad heads rc=%u\n", (unsigned)rc);

    // the stage functions on an empty batch: every stage returns before it would launch
    ppl::common::TensorShape empty_q(ppl::common::DATATYPE_FLOAT16, {0, num_heads, head_dim});
    ppl::common::TensorShape empty_k(ppl::common::DATATYPE_FLOAT16, {0, num_kv_heads, head_dim});
    pmx::dynamic_batching_multi_head_cache_attention idle;
    rc = idle.heuristic_prepare(device_prop, &empty_q, query, &empty_k, current_key, &empty_k, current_value, &mask_shape,
                                nullptr, seqstarts, kvstarts, cachestarts, start_pos, nullptr, true, 0, 0, 0, 0, layer_idx,
                                num_layer, num_heads, num_kv_heads, head_dim, 1, 128, cache_stride_s, cache_stride_l,
                                cache_stride_h, cache_stride_kv, 64, true, true, true, true, 1, 0, cache, scale, &empty_q, output);
    const hipStream_t stream = nullptr;
    printf("idle prepare rc=%u kvstore=%u decode=%u prefill=%u forward=%u\n", (unsigned)rc, (unsigned)idle.forward_kvstore(stream),
           (unsigned)idle.forward_decode(stream), (unsigned)idle.forward_prefill(stream), (unsigned)idle.forward(stream));

    // the neighbours of the operator, through the reference's prototypes
    const reorder_fn reorder = &pmx::kv_cache_reorder;
    const invert_reorder_fn invert_reorder = &pmx::kv_cache_invert_reorder;
    const rope_fn rope = &pmx::dynamic_batching_rotary_position_embedding;
    const linear_fn linear = &pmx::row_parallel_linear; // picks the overload with the reference's argument list
    (void)linear;
    pmx::Stride stride = {};
    stride.p_stride_cache = 128 * 128;
    stride.p_stride_scale = 128 * 32;
    printf("reorder(no pages)=%u invert(no pages)=%u\n",
           (unsigned)reorder(stream, cache, scale, seqstarts, stride, stride, 0, 32, 8, 128, 128, 8, 0, 1, output),
           (unsigned)invert_reorder(stream, output, seqstarts, stride, stride, 0, 32, 8, 128, 128, 8, 0, 1, cache, scale));
    printf("rope(empty batch)=%u\n",
           (unsigned)rope(stream, &query_shape, query, &key_shape, current_key, start_pos, seqstarts, 10000.f, 0, head_dim, 0,
                          num_heads, num_kv_heads, 1, 8192, pmx::rope_scaling::NONE, 1.f, &query_shape, query, &key_shape,
                          current_key));
    printf("kvcache(empty batch)=%u\n",
           (unsigned)pmx::dynamic_batching_key_value_cache(stream, &key_shape, current_key, &key_shape, current_value, seqstarts,
                                                           cachestarts, start_pos, 0, 1, num_layer, layer_idx, num_kv_heads,
                                                           head_dim, 1, 128, cache_stride_s, cache_stride_l, cache_stride_h,
                                                           cache_stride_kv, 64, cache, scale));
    // the projection behind the attention: the reference's argument list without its cuBLASLt / NCCL arguments
    ppl::common::TensorShape no_rows(ppl::common::DATATYPE_FLOAT16, {0, num_heads * head_dim});
    ppl::common::TensorShape weight_shape(ppl::common::DATATYPE_FLOAT16, {4096, num_heads * head_dim});
    ppl::common::TensorShape bias_shape(ppl::common::DATATYPE_FLOAT16, {4096});
    printf("linear(no rows)=%u linear(not parallel)=%u\n",
           (unsigned)pmx::row_parallel_linear(stream, &no_rows, output, &weight_shape, cache, &bias_shape, nullptr,
                                              num_heads * head_dim, 4096, true, 0, nullptr, &no_rows, query),
           (unsigned)pmx::row_parallel_linear(stream, &no_rows, output, &weight_shape, cache, &bias_shape, nullptr,
                                              num_heads * head_dim, 4096, false, 0, nullptr, &no_rows, query));
    // ... and with the reference's whole argument list (row_parallel_linear.h:28-46): handle, algorithm, communicator
    // and split buffer are accepted as a call site passes them; a communicator of two ranks is refused
    cublasLtHandle_t blas_handle = nullptr;
    cublasLtMatmulAlgo_t algo = {};
    ppl::common::NcclParam one_rank, two_ranks;
    two_ranks.size = 2;
    printf("linear_ref(no rows)=%u linear_ref(null comm)=%u linear_ref(two ranks)=%u\n",
           (unsigned)pmx::row_parallel_linear(stream, blas_handle, &algo, &no_rows, output, &weight_shape, cache, &bias_shape, nullptr,
                                              num_heads * head_dim, 4096, &one_rank, true, nullptr, 0, nullptr, &no_rows, query),
           (unsigned)pmx::row_parallel_linear(stream, blas_handle, nullptr, &no_rows, output, &weight_shape, cache, &bias_shape,
                                              nullptr, num_heads * head_dim, 4096, nullptr, true, nullptr, 0, nullptr, &no_rows, query),
           (unsigned)pmx::row_parallel_linear(stream, blas_handle, &algo, &no_rows, output, &weight_shape, cache, &bias_shape, nullptr,
                                              num_heads * head_dim, 4096, &two_ranks, true, nullptr, 0, nullptr, &no_rows, query));
    return 0;
}
