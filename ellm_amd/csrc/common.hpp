// Shared device helpers for the gfx950 attention kernels: storage-type traits,
// MFMA wrappers with their operand layouts, and small wave-level utilities.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace ellm {

constexpr int kHeadDim = 128;  // the reference kernel is hard-wired to 128 too
constexpr int kWave = 64;

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

struct F16 {};   // IEEE binary16 storage
struct BF16 {};  // bfloat16 storage

// ---- MFMA wrappers ---------------------------------------------------------
// Operands travel as raw 128-bit / 64-bit register groups (8 or 4 packed 16-bit
// values per lane).  Layouts (lane l of the 64-wide wave):
//   32x32x16: A[i][k], B[k][j]: i or j = l % 32, k = 8*(l/32) + 0..7
//             C[i][j]: j = l % 32, i = 8*(r/4) + 4*(l/32) + r%4 for register r of 16
//   16x16x32: A[i][k], B[k][j]: i or j = l % 16, k = 8*(l/16) + 0..7
//             C[i][j]: j = l % 16, i = 4*(l/16) + r for register r of 4
//   16x16x16: A[i][k], B[k][j]: i or j = l % 16, k = 4*(l/16) + 0..3; C as 16x16x32

template <typename T>
struct Mfma;

template <>
struct Mfma<F16> {
  typedef F16 storage;
  static __device__ __forceinline__ f32x16 m32x32x16(u32x4 a, u32x4 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a),
                                                  __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ f32x4 m16x16x32(u32x4 a, u32x4 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a),
                                                  __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ f32x4 m16x16x16(u32x2 a, u32x2 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(f16x4, a),
                                                 __builtin_bit_cast(f16x4, b), c, 0, 0, 0);
  }
  // two binary32 -> packed pair, round to nearest even (v_cvt_pk_f16_f32)
  static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
    f32x2 x = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(x, f16x2));
  }
  // acc + lo + hi of a packed pair, accumulated in binary32 (v_dot2c_f32_f16)
  static __device__ __forceinline__ float add_pair(uint32_t packed, float acc) {
    const f16x2 ones = {(_Float16)1.0f, (_Float16)1.0f};
    return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2, packed), ones, acc, false);
  }
  static __device__ __forceinline__ float to_float(uint16_t bits) {
    return (float)__builtin_bit_cast(_Float16, bits);
  }
};

template <>
struct Mfma<BF16> {
  typedef BF16 storage;
  static __device__ __forceinline__ f32x16 m32x32x16(u32x4 a, u32x4 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a),
                                                   __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ f32x4 m16x16x32(u32x4 a, u32x4 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a),
                                                   __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ f32x4 m16x16x16(u32x2 a, u32x2 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(s16x4, a),
                                                     __builtin_bit_cast(s16x4, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
    f32x2 x = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(x, bf16x2));
  }
  static __device__ __forceinline__ float add_pair(uint32_t packed, float acc) {
    const bf16x2 ones = {(__bf16)1.0f, (__bf16)1.0f};
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, packed), ones, acc, false);
  }
  static __device__ __forceinline__ float to_float(uint16_t bits) {
    return __builtin_bit_cast(float, (uint32_t)bits << 16);
  }
};

// ---- small utilities -------------------------------------------------------

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fast_log2(float x) { return __builtin_amdgcn_logf(x); }

__device__ __forceinline__ u32x4 load16(const void* p) { return *(const u32x4*)p; }
__device__ __forceinline__ void store16(void* p, u32x4 v) { *(u32x4*)p = v; }
// The same for bytes that are touched once (streamed rows): marked so that the caches do not keep them.
__device__ __forceinline__ u32x4 load16_once(const void* p) { return __builtin_nontemporal_load((const u32x4*)p); }
__device__ __forceinline__ void store16_once(void* p, u32x4 v) { __builtin_nontemporal_store(v, (u32x4*)p); }

// Exchange with the lane whose index differs in the given bit (16 or 32).
__device__ __forceinline__ float xor_shuffle(float v, int mask) { return __shfl_xor(v, mask, 64); }

// v_permlane32_swap exchanges the upper half of one register with the lower half
// of another; swapping a value with a copy of itself (in a second register: a
// register swapped with itself keeps its lower half) yields, in every lane l, the
// value of lane l % 32 in one register and of lane 32 + l % 32 in the other, i.e.
// the lane's own value and its partner's (lane l ^ 32), without a trip through LDS.
// Written as inline asm: with the builtin the optimiser folds max / add of the two
// results as if they were equal.  The s_nop pairs cover the VALU-write -> permlane
// read and permlane write -> VALU read wait states the compiler cannot see here.
__device__ __forceinline__ void swap_halves(float& a, float& b) {
  asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
}
__device__ __forceinline__ float max_with_partner_half(float v) {
  float a = v, b = v;
  swap_halves(a, b);
  return fmaxf(a, b);
}
__device__ __forceinline__ float sum_with_partner_half(float v) {
  float a = v, b = v;
  swap_halves(a, b);
  return a + b;
}

// Regroup packed 16-bit pairs: given four registers holding (x[k][2c], x[k][2c+1])
// for k = 0..3, return the two registers holding (x[0][e], x[1][e]) and
// (x[2][e], x[3][e]) for e = 2c (hi = false) or 2c+1 (hi = true).
__device__ __forceinline__ u32x2 gather_column(uint32_t r0, uint32_t r1, uint32_t r2, uint32_t r3,
                                               bool hi) {
  u32x2 o;
  if (hi) {
    o[0] = (r0 >> 16) | (r1 & 0xffff0000u);
    o[1] = (r2 >> 16) | (r3 & 0xffff0000u);
  } else {
    o[0] = (r0 & 0xffffu) | (r1 << 16);
    o[1] = (r2 & 0xffffu) | (r3 << 16);
  }
  return o;
}

// Element offset of the first K/V plane of a sequence: sequence x stride, or, for a cache
// whose sequences have different capacities, the sequence's entry of an offset table.
__device__ __forceinline__ size_t seq_plane_offset(const size_t* table, size_t stride, uint32_t seq) {
  return table ? table[seq] : (size_t)seq * stride;
}

// What the fused Q/K/V projection does to every finished query / key head row (reference:
// matmul_finalize_rmsnorm_rope_inplace_3x128, src/kernel/x86_64/f16_512/matmul_rms_complex.rs:76-96),
// on the eight consecutive elements a lane holds:
//   sum of squares of the lane's eight elements, in order, with fused multiply-adds;
//   y = x / (sqrt(mean of squares) + eps), eps added to the root (src/kernel/generic/rms_norm.rs:19);
//   (a, b) -> (a cos - b sin, a sin + b cos) with the four (cos, sin) pairs of `rope8`.
// The caller adds the lanes' sums of squares up to the head's 128 elements in between.
__device__ __forceinline__ float squares8(const float (&x)[8]) {
  float ss = 0.0f;
#pragma unroll
  for (int e = 0; e < 8; ++e) ss = fmaf(x[e], x[e], ss);
  return ss;
}
__device__ __forceinline__ float inverse_rms(float sum_of_squares, float eps) {
  return 1.0f / (sqrtf(sum_of_squares / (float)kHeadDim) + eps);
}
template <typename T>
__device__ __forceinline__ u32x4 scale_rotate_pack8(const float (&x)[8], float inv, u32x4 rope8) {
  u32x4 out;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const float cs = Mfma<T>::to_float((uint16_t)(rope8[e] & 0xffffu)), sn = Mfma<T>::to_float((uint16_t)(rope8[e] >> 16));
    const float y0 = x[2 * e] * inv, y1 = x[2 * e + 1] * inv;
    out[e] = Mfma<T>::pack2(y0 * cs - y1 * sn, y0 * sn + y1 * cs);
  }
  return out;
}

// The value lane - 1 of the same 16-lane row holds; 0 in the row's first lane (a data-parallel
// move inside the vector ALU, no trip through the LDS crossbar).
__device__ __forceinline__ float from_left_neighbour(float v) {
  constexpr int kRowShr1 = 0x111;
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), kRowShr1, 0xf, 0xf, true));
}

// One 128-wide key row as a stored 16-bit row, normalised and rotated the way the cache write
// does it (kv_append_norm_rope_kernel; the reference's scalar order, generic forms
// src/kernel/generic/rms_norm.rs:6-26 and complex_mul.rs:3-20):
//   y = x / (sqrt(mean(x^2)) + eps);  (e, f) = (a c - b d, a d + b c) for the interleaved pairs
//   (a, b) of y and (c, d) = (cos, sin) of the rotary row.
// Sixteen lanes own the row (lane c of the 16-lane row: elements 8 c .. 8 c + 7 in kraw, the
// same elements of the rotary row in rraw).  Binary32 with one rounding per operation and no
// contraction; the sum of squares runs through the 128 elements first to last: turn by turn
// every lane adds its eight squares to what its left neighbour held after the turn before, so
// lane c's value is final from turn c on and lane 15 ends with the whole sum, the same bits a
// sequential CPU loop produces.  Every lane of the wave must call this (row shifts, one shuffle).
template <typename T>
__device__ __forceinline__ u32x4 norm_rope_row16(u32x4 kraw, u32x4 rraw, float eps) {
#pragma clang fp contract(off)
  float x[8], sq[8];
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    x[2 * e] = Mfma<T>::to_float((uint16_t)(kraw[e] & 0xffffu));
    x[2 * e + 1] = Mfma<T>::to_float((uint16_t)(kraw[e] >> 16));
  }
#pragma unroll
  for (int e = 0; e < 8; ++e) sq[e] = x[e] * x[e];
  float mine = 0.0f;
#pragma unroll
  for (int l = 0; l < 16; ++l) {
    mine = from_left_neighbour(mine);
#pragma unroll
    for (int e = 0; e < 8; ++e) mine = mine + sq[e];
  }
  const float sum = __shfl(mine, 15, 16);
  const float variance = sum / (float)kHeadDim;
  const float rrms = 1.0f / (sqrtf(variance) + eps);
  u32x4 out;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const float a = x[2 * e] * rrms, bb = x[2 * e + 1] * rrms;
    const float cs = Mfma<T>::to_float((uint16_t)(rraw[e] & 0xffffu));
    const float sn = Mfma<T>::to_float((uint16_t)(rraw[e] >> 16));
    const float re = a * cs - bb * sn;
    const float im = a * sn + bb * cs;
    out[e] = Mfma<T>::pack2(re, im);
  }
  return out;
}

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

}  // namespace ellm
