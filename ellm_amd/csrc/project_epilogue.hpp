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

constexpr int kEpPitch = kHeadDim * 2 + 16;           // a 256-byte row in LDS
constexpr int kEpWaveBytes = 2 * 32 * kEpPitch;       // per wave: 32 output rows and 32 rows of the extra operand

typedef __attribute__((address_space(1))) u32x4 GlobalVec4;

// acc[nb][mb]: column block nb (32 columns) x token block mb (32 tokens) of head `hh`;
// `first_row` is the row of the activations that token block 0, lane row 0 stands for;
// `ep_rows` is the LDS byte address of kEpWaveBytes that belong to this wave alone.
// In the accumulator layout lane (j, g) holds, for token 32 mb + j, the
// columns 32 nb + 8 b + 4 g + (0..3) of the head: four consecutive columns = two rotation
// pairs = one 8-byte piece of the rotary row, of the residual row and of the output
// row; lanes l and l ^ 32 together own the token's 128 columns.
// Memory is touched in whole rows only, in both directions: a wave instruction moves four
// 256-byte rows (16 lanes a row), and LDS turns rows into the accumulator layout and back.
// (Fetching the extra operand in the accumulator layout directly, 8 bytes a lane from 32
// different rows per instruction, cost the vector cache 32 line look-ups an instruction and
// 200 cycles each: 1.3 us a token block on a wave that has nothing else to run.)  Which row
// a lane moves is lane / 16 + 4 i; the row's address comes from the lane that owns the token
// through a lane permute.  The extra operand (table or residual) of token block mb + 2 is
// requested while block mb is worked on, ahead of block mb's stores.
// One code path: a head that is not normalised and rotated runs the same arithmetic
// with scale 1 and the rotation (cos, sin) = (1, 0), which leaves every value as it is.
// HeadRows: where the rows of one head x 32 MB tokens go and what is combined with them, plus
// the extra operand of token block 0, already requested: a kernel with registers to spare calls
// prepare_head() ahead of its main loop, so that neither the positions nor the first table /
// residual rows are waited for after it.
template <int MB>
struct HeadRows {
  uint16_t* out_row[MB];        // this lane's token: destination row (g == 0 and g == 1 alike)
  const uint16_t* ext_row[MB];  // ... and row of the extra operand; null: none (scale 1, no rotation)
  bool present;    // false: the head lies beyond the last one (odd head count), nothing to do
  bool finalize;   // normalise + rotate
  u32x4 ext0[8];   // token block 0's extra rows as fetched: piece lane % 16 of rows lane / 16 + 4 i
};

// The 64-bit value that lane `from` holds (every lane names its own source lane).
__device__ __forceinline__ uint64_t from_lane(uint64_t v, int from) {
  const uint32_t lo = (uint32_t)__builtin_amdgcn_ds_bpermute(4 * from, (int)(uint32_t)v);
  const uint32_t hi = (uint32_t)__builtin_amdgcn_ds_bpermute(4 * from, (int)(uint32_t)(v >> 32));
  return ((uint64_t)hi << 32) | lo;
}

// The residual rows of the 128-token-a-wave tiles (thousands of rows a call, each piece read by
// one workgroup) are marked non-temporal: 1.5 % on 32768 rows; with the smaller tiles' few
// hundred rows, which their producer may have left in a cache, the mark cost 1 %.
template <int MODE, int MB>
constexpr bool kStreamedResidual = MODE == kModeAdd && MB >= 4;

// Rows lane / 16 + 4 i, i = 0..7, of the extra operand of one token block; rows without one
// read as (1, 0) pairs.  ONCE: rows nobody reads again, marked non-temporal.
template <typename S, bool ONCE>
__device__ __forceinline__ void fetch_ext_rows(const uint16_t* my_row, int lane, u32x4 (&v)[8]) {
  const uint32_t one_zero = Mfma<S>::pack2(1.0f, 0.0f);
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const uint64_t row = from_lane((uint64_t)my_row, 4 * i + (lane >> 4));
    v[i] = u32x4{one_zero, one_zero, one_zero, one_zero};
    if (row) {
      if constexpr (ONCE)
        v[i] = __builtin_nontemporal_load((const GlobalVec4*)(row + 16 * (lane & 15)));
      else
        v[i] = *(const GlobalVec4*)(row + 16 * (lane & 15));
    }
  }
}

template <typename S, int MODE, int MB>
__device__ __forceinline__ HeadRows<MB> prepare_head(const ProjectKernelArgs& p, uint32_t hh,
                                                     uint32_t first_row, int lane) {
  HeadRows<MB> h;
  const int j = lane & 31;
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
    const bool live = h.present && R < p.rows && b < p.batch;
    uint32_t pos = t;
    if (p.positions)
      pos += live ? min(p.positions[b], p.max_start) : 0u;
    else
      pos += p.position_index;
    const size_t col = hs * kHeadDim;
    h.out_row[mb] = nullptr;
    h.ext_row[mb] = nullptr;
    if (live) {
      h.out_row[mb] = (seg == 0) ? dst + (size_t)R * p.ld0 + col : dst + kv_row_offset(p, b, hs, pos);
      if (MODE == kModeAdd)
        h.ext_row[mb] = p.residual + (size_t)R * p.ld0 + col;
      else if (h.finalize)
        h.ext_row[mb] = p.rope + (size_t)pos * p.rope_pos_stride + (size_t)hs * p.rope_head_stride;
    }
  }
  fetch_ext_rows<S, kStreamedResidual<MODE, MB>>(h.ext_row[0], lane, h.ext0);
  return h;
}

template <typename S, int MODE, int MB>
__device__ __forceinline__ void finish_head(const ProjectKernelArgs& p, f32x16 (&acc)[4][MB],
                                            const HeadRows<MB>& h, uint32_t ep_rows, int lane) {
  using M = Mfma<S>;
  const int j = lane & 31, g = lane >> 5;
  if (!h.present) return;
  const bool finalize = h.finalize;
  const uint32_t ep_ext = ep_rows + 32 * kEpPitch;
  // this lane's place as a mover of whole rows (row lane / 16 + 4 i, piece lane % 16) and as the
  // owner of token j (8-byte pieces at columns 32 nb + 8 b + 4 g)
  const uint32_t row_piece = (lane >> 4) * kEpPitch + 16 * (lane & 15);
  const uint32_t own_piece = j * kEpPitch + 8 * g;
  u32x4 raw[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) raw[i] = h.ext0[i];
  // the extra rows of a block go into LDS as soon as the block before has read its own out of it,
  // and the block after is requested: both ahead of that block's stores, so that a wait for
  // the rows never includes stores (the compiler cannot count conditional stores and waits for all)
  auto stage_ext = [&](int next) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < 8; ++i) *(LdsVec4*)(ep_ext + row_piece + 4 * i * kEpPitch) = raw[i];
    if (next < MB) fetch_ext_rows<S, kStreamedResidual<MODE, MB>>(h.ext_row[next < MB ? next : 0], lane, raw);
  };
  stage_ext(1);
  static_for<MB>([&](auto mb_) {
    constexpr int mb = decltype(mb_)::value;
    __builtin_amdgcn_sched_barrier(0);  // one token block's accumulators at a time leave the AGPRs
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
    u32x2 ext[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) ext[i] = *(const LdsVec2*)(ep_ext + own_piece + 2 * (32 * (i >> 2) + 8 * (i & 3)));
    u32x2 packed[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int nb = i >> 2, b4 = i & 3;
      float o0 = acc[nb][mb][4 * b4], o1 = acc[nb][mb][4 * b4 + 1];
      float o2 = acc[nb][mb][4 * b4 + 2], o3 = acc[nb][mb][4 * b4 + 3];
      const u32x2 rr = ext[i];
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
    // out through LDS: the owner of a token leaves its row there, the movers of whole rows pick
    // up all eight of theirs before the first store
#pragma unroll
    for (int i = 0; i < 16; ++i)
      *(LdsVec2*)(ep_rows + own_piece + 2 * (32 * (i >> 2) + 8 * (i & 3))) = packed[i];
    if constexpr (mb + 1 < MB) stage_ext(mb + 2);
    uint64_t to[8];
    u32x4 v[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      to[i] = from_lane((uint64_t)h.out_row[mb], 4 * i + (lane >> 4));   // 0: nothing to write
      v[i] = *(const LdsVec4*)(ep_rows + row_piece + 4 * i * kEpPitch);
    }
#pragma unroll
    for (int i = 0; i < 8; ++i)
      if (to[i]) __builtin_nontemporal_store(v[i], (GlobalVec4*)(to[i] + 16 * (lane & 15)));
  });
}

}  // namespace proj
}  // namespace ellm
