// Epilogue shared by the MFMA tile kernels of the projections: a wave that holds one head
// (128 output columns) of 32 * MB tokens as transposed 32x32 accumulator blocks finishes
// the head rows (RMS norm + rotary rotation, or residual add), rounds them and writes
// them to their destinations.
#pragma once

#include "project_common.hpp"

namespace ellm {
namespace proj {

typedef __attribute__((address_space(3))) u32x4 LdsVec4;
typedef __attribute__((address_space(3))) u32x2 LdsVec2;
typedef __attribute__((address_space(3))) uint64_t LdsU64;

constexpr int kEpPitch = kHeadDim * 2 + 16;           // output row in LDS
constexpr int kEpWaveBytes = 32 * kEpPitch + 32 * 8;  // 32 rows and their destinations, per wave

// acc[nb][mb]: column block nb (32 columns) x token block mb (32 tokens) of head `hh`;
// `first_row` is the row of the activations that token block 0, lane row 0 stands for;
// `ep_rows` is the LDS byte address of kEpWaveBytes that belong to this wave alone.
// In the accumulator layout lane (j, g) holds, for token 32 mb + j, the
// columns 32 nb + 8 b + 4 g + (0..3) of the head: four consecutive columns = two rotation
// pairs = one 8-byte piece of the rotary row, of the residual row and of the output
// row; lanes l and l ^ 32 together own the token's 128 columns.  The extra operand
// (table or residual) of token block mb + 1 is requested before block mb is worked on.
// One code path: a head that is not normalised and rotated runs the same arithmetic
// with scale 1 and the rotation (cos, sin) = (1, 0), which leaves every value as it is.
// Where the rows of one head x 32 MB tokens go and what is combined with them, plus the extra
// operand of token block 0, already requested: a kernel with registers to spare calls
// prepare_head() ahead of its main loop, so that neither the positions nor the first table /
// residual rows are waited for after it.
template <int MB>
struct HeadRows {
  uint16_t* out_row[MB];
  const uint16_t* ext_row[MB];
  bool live[MB];
  bool present;    // false: the head lies beyond the last one (odd head count), nothing to do
  bool finalize;   // normalise + rotate
  u32x2 ext0[16];
};

template <typename S, int MODE, int MB>
__device__ __forceinline__ HeadRows<MB> prepare_head(const ProjectKernelArgs& p, uint32_t hh,
                                                     uint32_t first_row, int lane) {
  using M = Mfma<S>;
  HeadRows<MB> h;
  const int j = lane & 31, g = lane >> 5;
  const uint32_t heads_total = p.heads0 + 2 * p.heads_kv;
  h.present = hh < heads_total;
  const uint32_t seg = (hh < p.heads0) ? 0u : (hh < p.heads0 + p.heads_kv ? 1u : 2u);
  const uint32_t hs = hh - (seg == 0 ? 0u : (seg == 1 ? p.heads0 : p.heads0 + p.heads_kv));
  h.finalize = MODE == kModeQkv && ((seg == 1) || (seg == 0 && p.finalize0));
  uint16_t* const dst = (seg == 0) ? p.out0 : (seg == 1 ? p.k_out : p.v_out);
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) {
    const uint32_t R = first_row + 32 * mb + j;
    const uint32_t t = R / p.batch_pitch, b = R % p.batch_pitch;
    h.live[mb] = h.present && R < p.rows && b < p.batch;
    uint32_t pos = t;
    if (p.positions)
      pos += h.live[mb] ? min(p.positions[b], p.max_start) : 0u;
    else
      pos += p.position_index;
    const size_t col = hs * kHeadDim;
    if (seg == 0)
      h.out_row[mb] = dst + (size_t)R * p.ld0 + col;
    else
      h.out_row[mb] = dst + (h.live[mb] ? kv_row_offset(p, b, hs, pos) : (size_t)0);
    if (MODE == kModeQkv)
      h.ext_row[mb] = p.rope + (size_t)pos * p.rope_pos_stride + (size_t)hs * p.rope_head_stride + 4 * g;
    else
      h.ext_row[mb] = p.residual + (size_t)R * p.ld0 + col + 4 * g;
  }
  const uint32_t one_zero = M::pack2(1.0f, 0.0f);
  if ((MODE == kModeAdd || h.finalize) && h.live[0]) {
#pragma unroll
    for (int i = 0; i < 16; ++i) h.ext0[i] = *(const u32x2*)(h.ext_row[0] + 32 * (i >> 2) + 8 * (i & 3));
  } else {
#pragma unroll
    for (int i = 0; i < 16; ++i) h.ext0[i] = u32x2{one_zero, one_zero};
  }
  return h;
}

template <typename S, int MODE, int MB>
__device__ __forceinline__ void finish_head(const ProjectKernelArgs& p, f32x16 (&acc)[4][MB],
                                            const HeadRows<MB>& h, uint32_t ep_rows, int lane) {
  using M = Mfma<S>;
  const int j = lane & 31, g = lane >> 5;
  if (!h.present) return;
  const bool finalize = h.finalize;
  const auto& out_row = h.out_row;
  const auto& ext_row = h.ext_row;
  const auto& live = h.live;
  const uint32_t ep_table = ep_rows + 32 * kEpPitch;
  const uint32_t one_zero = M::pack2(1.0f, 0.0f);
  u32x2 ext[2][16];
  auto fetch_ext = [&](auto set, int mb) {
    if ((MODE == kModeAdd || finalize) && live[mb]) {
#pragma unroll
      for (int i = 0; i < 16; ++i) ext[set][i] = *(const u32x2*)(ext_row[mb] + 32 * (i >> 2) + 8 * (i & 3));
    } else {
#pragma unroll
      for (int i = 0; i < 16; ++i) ext[set][i] = u32x2{one_zero, one_zero};
    }
  };
#pragma unroll
  for (int i = 0; i < 16; ++i) ext[0][i] = h.ext0[i];
  static_for<MB>([&](auto mb_) {
    constexpr int mb = decltype(mb_)::value;
    constexpr int set = mb & 1;
    __builtin_amdgcn_sched_barrier(0);  // one token block's accumulators at a time leave the AGPRs
    if constexpr (mb + 1 < MB) fetch_ext(std::integral_constant<int, 1 - set>{}, mb + 1);
    float inv = 1.0f;
    if (MODE == kModeQkv) {
      float ss = 0.0f;
#pragma unroll
      for (int nb = 0; nb < 4; ++nb)
#pragma unroll
        for (int r = 0; r < 16; ++r) ss = fmaf(acc[nb][mb][r], acc[nb][mb][r], ss);
      ss = sum_with_partner_half(ss);
      inv = finalize ? 1.0f / (sqrtf(ss / (float)kHeadDim) + p.eps) : 1.0f;
    }
    u32x2 packed[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int nb = i >> 2, b4 = i & 3;
      float o0 = acc[nb][mb][4 * b4], o1 = acc[nb][mb][4 * b4 + 1];
      float o2 = acc[nb][mb][4 * b4 + 2], o3 = acc[nb][mb][4 * b4 + 3];
      const u32x2 rr = ext[set][i];
      const float e0 = M::to_float((uint16_t)(rr[0] & 0xffffu)), e1 = M::to_float((uint16_t)(rr[0] >> 16));
      const float e2 = M::to_float((uint16_t)(rr[1] & 0xffffu)), e3 = M::to_float((uint16_t)(rr[1] >> 16));
      if (MODE == kModeQkv) {
        const float y0 = o0 * inv, y1 = o1 * inv, y2 = o2 * inv, y3 = o3 * inv;
        o0 = y0 * e0 - y1 * e1;
        o1 = y0 * e1 + y1 * e0;
        o2 = y2 * e2 - y3 * e3;
        o3 = y2 * e3 + y3 * e2;
      } else {
        o0 += e0;
        o1 += e1;
        o2 += e2;
        o3 += e3;
      }
      packed[i] = u32x2{M::pack2(o0, o1), M::pack2(o2, o3)};
    }
    // out through LDS so that a store instruction covers whole 256-byte rows: the lane
    // that owns token j also leaves the row's destination (0: nothing to write)
    if (g == 0) *(LdsU64*)(ep_table + 8 * j) = live[mb] ? (uint64_t)out_row[mb] : 0ull;
#pragma unroll
    for (int i = 0; i < 16; ++i)
      *(LdsVec2*)(ep_rows + j * kEpPitch + 2 * (32 * (i >> 2) + 8 * (i & 3) + 4 * g)) = packed[i];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const uint32_t row = 4 * i + (lane >> 4);
      uint16_t* const to = (uint16_t*)*(const LdsU64*)(ep_table + 8 * row);
      const u32x4 v = *(const LdsVec4*)(ep_rows + row * kEpPitch + 16 * (lane & 15));
      if (to) store16(to + 8 * (lane & 15), v);
    }
  });
}

}  // namespace proj
}  // namespace ellm
