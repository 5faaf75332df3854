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
    uint32_t n_kv_heads, KvLayout layout, uint32_t position_index) {
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
    const size_t dst = seq_plane_offset(layout.seq_offsets, layout.stride_seq, b) +
                       (size_t)h * layout.stride_head + (size_t)(position_index + t) * kHeadDim + 8 * c;
    store16_once(k_dst + dst, load16_once(k_src + src));
    store16_once(v_dst + dst, load16_once(v_src + src));
  }
}

// The same write with the key rows normalised and rotated on the way in (what the
// reference's fused projection does to a finished 128-wide head column,
// src/kernel/x86_64/f16_512/matmul_rms_complex.rs:76-96, generic forms
// src/kernel/generic/rms_norm.rs:6-26 and complex_mul.rs:3-20):
//   y = x / (sqrt(mean(x^2)) + eps);  (e, f) = (a c - b d, a d + b c) for the
//   interleaved pairs (a, b) of y and (c, d) = (cos, sin) of the rotary row of
//   the token's position.
// Sixteen lanes own one row (8 elements each); the arithmetic is norm_rope_row16 (common.hpp):
// binary32, one rounding per operation, the reference's scalar order, so the stored rows are
// the bits a sequential CPU loop produces.
template <typename T>
__global__ __launch_bounds__(256) void kv_append_norm_rope_kernel(
    uint16_t* __restrict__ k_dst, uint16_t* __restrict__ v_dst, const uint16_t* __restrict__ k_src,
    const uint16_t* __restrict__ v_src, const uint16_t* __restrict__ rope,
    const uint32_t* __restrict__ positions, uint32_t n_tokens, uint32_t batch,
    uint32_t src_batch_pitch, uint32_t n_kv_heads, KvLayout layout, uint32_t position_index,
    uint32_t max_start, float eps) {
  const uint32_t c = threadIdx.x & 15;
  const size_t rows = (size_t)n_tokens * batch * n_kv_heads;
  // every lane of a wave runs the same number of trips: the loop holds cross-lane reads
  const size_t rows_per_pass = (size_t)gridDim.x * (blockDim.x >> 4);
  const size_t passes = (rows + rows_per_pass - 1) / rows_per_pass;
  for (size_t pass = 0; pass < passes; ++pass) {
    const size_t row = pass * rows_per_pass + (size_t)blockIdx.x * (blockDim.x >> 4) + (threadIdx.x >> 4);
    const bool live = row < rows;
    size_t r = live ? row : 0;
    const uint32_t h = r % n_kv_heads;
    r /= n_kv_heads;
    const uint32_t b = r % batch;
    const uint32_t t = r / batch;
    const uint32_t start = positions ? min(positions[b], max_start) : position_index;
    const uint32_t pos = start + t;
    const size_t src = (((size_t)t * src_batch_pitch + b) * n_kv_heads + h) * kHeadDim + 8 * c;
    // (per-sequence capacities, where the cache has them, bound the row written: a start
    // position beyond a short sequence's planes must not reach into its neighbour's)
    const uint32_t pos_dst = layout.seq_caps ? min(pos, layout.seq_caps[b] - 1) : pos;
    const size_t dst = seq_plane_offset(layout.seq_offsets, layout.stride_seq, b) +
                       (size_t)h * layout.stride_head + (size_t)pos_dst * kHeadDim + 8 * c;
    const u32x4 kraw = load16_once(k_src + src);
    const u32x4 vraw = load16_once(v_src + src);
    const u32x4 rraw = load16(rope + (size_t)pos * kHeadDim + 8 * c);
    const u32x4 out = norm_rope_row16<typename T::storage>(kraw, rraw, eps);
    if (live) {
      store16_once(k_dst + dst, out);
      store16_once(v_dst + dst, vraw);
    }
  }
}

__global__ void fill_u32_kernel(uint32_t* p, size_t n, uint32_t value) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = value;
}

__global__ void positions_advance_kernel(uint32_t* positions, uint32_t n, uint32_t by) {
  const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) positions[i] += by;
}

}  // namespace

hipError_t launch_fill_u32(uint32_t* p, size_t n, uint32_t value, hipStream_t stream) {
  if (n == 0) return hipSuccess;
  hipLaunchKernelGGL(fill_u32_kernel, dim3((uint32_t)((n + 255) / 256)), dim3(256), 0, stream, p, n, value);
  return hipGetLastError();
}

hipError_t launch_positions_advance(uint32_t* positions, uint32_t n, uint32_t by,
                                    hipStream_t stream) {
  if (n == 0) return hipSuccess;
  hipLaunchKernelGGL(positions_advance_kernel, dim3((n + 255) / 256), dim3(256), 0, stream,
                     positions, n, by);
  return hipGetLastError();
}

hipError_t launch_kv_append_norm_rope(void* k_dst, void* v_dst, const void* k_src,
                                      const void* v_src, const void* rope,
                                      const uint32_t* positions, uint32_t n_tokens, uint32_t batch,
                                      uint32_t src_batch_pitch, uint32_t n_kv_heads,
                                      const KvLayout& layout, uint32_t position_index,
                                      uint32_t max_start, float eps, int dtype,
                                      hipStream_t stream) {
  const size_t rows = (size_t)n_tokens * batch * n_kv_heads;
  if (rows == 0) return hipSuccess;
  size_t blocks = (rows + 15) / 16;
  if (blocks > 16384) blocks = 16384;
  auto go = [&](auto kernel) {
    hipLaunchKernelGGL(kernel, dim3((uint32_t)blocks), dim3(256), 0, stream, (uint16_t*)k_dst,
                       (uint16_t*)v_dst, (const uint16_t*)k_src, (const uint16_t*)v_src,
                       (const uint16_t*)rope, positions, n_tokens, batch, src_batch_pitch,
                       n_kv_heads, layout, position_index, max_start, eps);
  };
  if (dtype == 0)
    go(kv_append_norm_rope_kernel<Mfma<F16>>);
  else
    go(kv_append_norm_rope_kernel<Mfma<BF16>>);
  return hipGetLastError();
}

hipError_t launch_kv_append(void* k_dst, void* v_dst, const void* k_src, const void* v_src,
                            uint32_t n_tokens, uint32_t batch, uint32_t src_batch_pitch,
                            uint32_t n_kv_heads, const KvLayout& layout, uint32_t position_index,
                            hipStream_t stream) {
  const size_t total = (size_t)n_tokens * batch * n_kv_heads * 16;
  if (total == 0) return hipSuccess;
  size_t blocks = (total + 255) / 256;
  if (blocks > 65536) blocks = 65536;
  hipLaunchKernelGGL(kv_append_kernel, dim3((uint32_t)blocks), dim3(256), 0, stream,
                     (uint16_t*)k_dst, (uint16_t*)v_dst, (const uint16_t*)k_src,
                     (const uint16_t*)v_src, n_tokens, batch, src_batch_pitch, n_kv_heads, layout,
                     position_index);
  return hipGetLastError();
}

}  // namespace ellm
