// Shared by the two projection kernels (tile kernel for many rows, streaming kernel
// for a few rows): kernel arguments and small helpers.
#pragma once

#include <type_traits>

#include "common.hpp"
#include "kernels.hpp"

namespace ellm {
namespace proj {

constexpr int kBufFlags = 0x00020000;  // raw buffer of 32-bit data, no swizzle

struct ProjectKernelArgs {
  const uint16_t* x;         // [rows][K]
  const uint16_t* w[3];      // column segments 0 (query / plain), 1 (key), 2 (value): [heads * 128][K]
  uint16_t* out0;            // segment 0 destination, row-major [rows][ld0]
  const uint16_t* residual;  // added to segment 0 (same layout), may be null
  uint16_t* k_out;
  uint16_t* v_out;
  const uint16_t* rope;
  const uint32_t* positions;
  const size_t* seq_offsets;   // per-sequence plane offsets (null: sequence x kv_stride_seq)
  const uint32_t* seq_caps;    // per-sequence capacities (null: none to clamp to)
  size_t kv_stride_seq, kv_stride_head, kv_stride_pos;  // elements
  uint32_t ld0;
  uint32_t rope_pos_stride, rope_head_stride;           // elements
  uint32_t K, rows, batch_pitch, batch;
  uint32_t heads0, heads_kv;
  uint32_t tiles_m, tiles_n;
  uint32_t position_index, max_start;
  uint32_t finalize0;        // segment 0 rows are normalised and rotated
  float eps;
};

// Element offset of the K/V row of (sequence b, kv head hs, position pos) in k_out / v_out.
__device__ __forceinline__ size_t kv_row_offset(const ProjectKernelArgs& p, uint32_t b, uint32_t hs,
                                                uint32_t pos) {
  if (p.seq_caps) pos = min(pos, p.seq_caps[b] - 1);
  return seq_plane_offset(p.seq_offsets, p.kv_stride_seq, b) + (size_t)hs * p.kv_stride_head +
         (size_t)pos * p.kv_stride_pos;
}

template <int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
  if constexpr (N > 0) {
    static_for<N - 1>(f);
    f(std::integral_constant<int, N - 1>{});
  }
}

__device__ __forceinline__ uint64_t uniform64(const void* p) {
  const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(uint64_t)p);
  const uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)((uint64_t)p >> 32));
  return ((uint64_t)hi << 32) | (uint64_t)lo;
}

constexpr int kModeQkv = 0;  // heads normalised + rotated (or passed through), K/V to token coordinates
constexpr int kModeAdd = 1;  // plain product plus a residual of the output's layout
constexpr int kModeRaw = 2;  // the binary32 sums of every column to the workspace, [row][column]: a fused
                             // single-token step, whose attention kernel finishes the rows (few-rows kernel only)

// Streaming kernel for a few rows (project_small.hip).  It would take up to 128 rows, but from
// about 64 on one 128-token tile per head (project_mid.hip) is faster: measured for the
// 2048 -> 5120 product 19 / 29 us at 64 / 128 rows against a flat 18.5 us.
constexpr uint32_t kSmallRowsMax = 64;
hipError_t small_prepare();
bool small_kernel_takes(uint32_t rows, uint32_t K);
size_t small_workspace_floats(uint32_t heads, uint32_t K);
// mode: kModeQkv, kModeAdd or kModeRaw
hipError_t launch_project_small(const ProjectKernelArgs& p, float* ws, uint32_t* counters, int dtype,
                                int mode, hipStream_t stream);

// Tile kernel with 128-token x one-head tiles (project_mid.hip), for row counts at which
// the 256 x 256 tiles are fewer than the compute units.
hipError_t mid_prepare();
// token_blocks: 1 = 128-token tiles, 2 = 256-token tiles
hipError_t launch_project_mid(ProjectKernelArgs p, uint32_t token_blocks, int dtype, bool add,
                              hipStream_t stream);

}  // namespace proj
}  // namespace ellm
