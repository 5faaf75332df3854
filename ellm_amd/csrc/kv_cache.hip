// In-place K/V cache writes: [token][sequence][kv_head][128] rows produced by the
// projection go to their token coordinates in the dimension-first cache
// [sequence][kv_head][position][128].  The reference only hints at such a write
// (the output_to_kv flag, src/compiler/zip_map/complex_zip.rs:92-98); its live
// graph re-views the projection output instead (src/qwen3_moe/attention.rs:149-166).
#include "common.hpp"
#include "kernels.hpp"

namespace ellm {
namespace {

__global__ __launch_bounds__(256) void kv_append_kernel(
    uint16_t* __restrict__ k_dst, uint16_t* __restrict__ v_dst, const uint16_t* __restrict__ k_src,
    const uint16_t* __restrict__ v_src, uint32_t n_tokens, uint32_t batch, uint32_t src_batch_pitch,
    uint32_t n_kv_heads, uint32_t capacity, uint32_t position_index) {
  // one thread per 16-byte chunk; 16 chunks per 128-element row
  const size_t total = (size_t)n_tokens * batch * n_kv_heads * 16;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total;
       i += (size_t)gridDim.x * blockDim.x) {
    const uint32_t c = i & 15;
    size_t r = i >> 4;
    const uint32_t h = r % n_kv_heads;
    r /= n_kv_heads;
    const uint32_t b = r % batch;
    const uint32_t t = r / batch;
    const size_t src = (((size_t)t * src_batch_pitch + b) * n_kv_heads + h) * kHeadDim + 8 * c;
    const size_t dst =
        (((size_t)b * n_kv_heads + h) * capacity + position_index + t) * kHeadDim + 8 * c;
    store16(k_dst + dst, load16(k_src + src));
    store16(v_dst + dst, load16(v_src + src));
  }
}

}  // namespace

hipError_t launch_kv_append(void* k_dst, void* v_dst, const void* k_src, const void* v_src,
                            uint32_t n_tokens, uint32_t batch, uint32_t src_batch_pitch,
                            uint32_t n_kv_heads, uint32_t capacity, uint32_t position_index,
                            hipStream_t stream) {
  const size_t total = (size_t)n_tokens * batch * n_kv_heads * 16;
  if (total == 0) return hipSuccess;
  size_t blocks = (total + 255) / 256;
  if (blocks > 65536) blocks = 65536;
  hipLaunchKernelGGL(kv_append_kernel, dim3((uint32_t)blocks), dim3(256), 0, stream,
                     (uint16_t*)k_dst, (uint16_t*)v_dst, (const uint16_t*)k_src,
                     (const uint16_t*)v_src, n_tokens, batch, src_batch_pitch, n_kv_heads, capacity,
                     position_index);
  return hipGetLastError();
}

}  // namespace ellm
