// Gather / scatter of whole int8 KV pages with their scales between the cache and a
// contiguous "outer" buffer, for gfx950.
//
// Semantics follow the reference's kv_cache_reorder / kv_cache_invert_reorder
// (src/ppl/kernel/llm/cuda/pmx/kv_cache_reorder.cu:24-65, 103-144): both tensors are
// addressed as bytes through five strides (layer, K/V plane, kv head, token, byte); the
// cache side adds page_id * head_dim * row_bytes (the reference takes its threads-per-row,
// head_dim, as the tokens of a page, kv_cache_reorder.cu:44), the outer side adds the slot
// offset (page_cache_bytes + page_scale_bytes) * tp_size * slot plus this rank's share
// (kv_cache_reorder.cu:50, 61).  The reference moves one byte per thread; here a lane moves
// 16 bytes whenever both byte strides are 1 and everything else is 16-byte aligned.
#include "device_common.h"
#include "launch_params.h"

namespace pmxhip {

template <int VEC>
__global__ __launch_bounds__(256) void page_copy_kernel(const PageCopyLaunch a)
{
    const int64_t row_units = a.row_bytes / VEC;
    const int64_t total = a.pages * a.layers * 2 * a.kv_heads * a.tokens * row_units;
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (int64_t)gridDim.x * blockDim.x) {
        int64_t r = idx;
        const int64_t w = r % row_units; r /= row_units;
        const int64_t t = r % a.tokens; r /= a.tokens;
        const int64_t h = r % a.kv_heads; r /= a.kv_heads;
        const int64_t kv = r & 1; r >>= 1;
        const int64_t l = r % a.layers;
        const int64_t slot = r / a.layers;
        const int64_t page = a.page_ids[slot];
        const int64_t src = slot * a.src_slot_stride + page * a.src_page_stride + l * a.src_stride[0] + kv * a.src_stride[1] +
                            h * a.src_stride[2] + t * a.src_stride[3] + w * VEC * a.src_stride[4];
        const int64_t dst = slot * a.dst_slot_stride + page * a.dst_page_stride + l * a.dst_stride[0] + kv * a.dst_stride[1] +
                            h * a.dst_stride[2] + t * a.dst_stride[3] + w * VEC * a.dst_stride[4];
        if (VEC == 16) *(u32x4*)(a.dst + dst) = *(const u32x4*)(a.src + src);
        else a.dst[dst] = a.src[src];
    }
}

static bool multiple_of_16(int64_t v) { return (v & 15) == 0; }

void launch_page_copy(const PageCopyLaunch& a, hipStream_t stream)
{
    bool vec = a.src_stride[4] == 1 && a.dst_stride[4] == 1 && multiple_of_16(a.row_bytes) &&
               multiple_of_16((int64_t)(uintptr_t)a.src) && multiple_of_16((int64_t)(uintptr_t)a.dst) &&
               multiple_of_16(a.src_slot_stride) && multiple_of_16(a.dst_slot_stride) &&
               multiple_of_16(a.src_page_stride) && multiple_of_16(a.dst_page_stride);
    for (int i = 0; i < 4; ++i) vec = vec && multiple_of_16(a.src_stride[i]) && multiple_of_16(a.dst_stride[i]);
    const int64_t units = a.pages * a.layers * 2 * a.kv_heads * a.tokens * (a.row_bytes / (vec ? 16 : 1));
    if (units <= 0) return;
    int64_t blocks = (units + 255) / 256;
    if (blocks > 256 * 32) blocks = 256 * 32; // grid-stride beyond 32 workgroups per CU
    if (vec) hipLaunchKernelGGL(page_copy_kernel<16>, dim3((unsigned)blocks), dim3(256), 0, stream, a);
    else hipLaunchKernelGGL(page_copy_kernel<1>, dim3((unsigned)blocks), dim3(256), 0, stream, a);
}

} // namespace pmxhip
