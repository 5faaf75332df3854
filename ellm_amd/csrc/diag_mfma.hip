// Diagnostic, not part of the attention library: what the matrix pipe of this part
// delivers on given operand VALUES when nothing else competes with it.  bench.py runs it
// beside the chunk-attention benchmark so that "fraction of what an MFMA stream sustains on
// this data" is a number timed in the same run on the same box, not an assumption: on
// dense random 16-bit operands the part lowers its clock under a pure MFMA stream, and the
// published peak is not reachable by any kernel on such data.
//
// One launch: every compute unit runs four waves (one per SIMD); a wave issues
// iters x 32 v_mfma_f32_32x32x16 on four independent accumulators, no global memory
// access in the loop.
//   mode 0: both operands stay in registers;
//   mode 1: the A operand of every MFMA is read from LDS (one ds_read_b128 per MFMA), which
//           is what a wave that owns 32 query rows has to do for its K and V fragments;
//   mode 2: mode 1 plus, per MFMA, the vector work a soft-max of the same tile shape costs
//           (per 32 MFMAs: 32 exp2, 64 fused multiply-adds, 32 max, 32 adds, 16 packing
//           conversions, 32 multiplies = 208 vector instructions), dealt out between the
//           MFMAs of the same wave: the instruction mix of the chunk-attention kernel with
//           nothing to wait for, i.e. what a perfect schedule of that mix would sustain.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/ellm_diag.h"

namespace {

typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef __bf16 b8 __attribute__((ext_vector_type(8)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __attribute__((address_space(3))) volatile u32x4 VolatileLdsU32x4;

template <int DT>
__device__ __forceinline__ f32x16 mfma(u32x4 a, u32x4 b, f32x16 c) {
  if constexpr (DT == 0)
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(h8, a), __builtin_bit_cast(h8, b), c,
                                                  0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(b8, a), __builtin_bit_cast(b8, b),
                                                   c, 0, 0, 0);
}

// The vector instructions one MFMA's share of a soft-max costs: exp2, fused multiply-add,
// max, add, multiply and (every other call) a packing conversion, on values that neither
// overflow nor vanish however long the loop runs.
__device__ __forceinline__ void vector_work(float (&x)[8], int i) {
  float& u = x[i & 7];
  float& w = x[(i + 3) & 7];
  const float e = __builtin_amdgcn_exp2f(-u);          // in [0.5, 1)
  const float f = __builtin_fmaf(e, 0.75f, 0.125f);    // in [0.5, 0.875)
  const float m = fmaxf(f, w * 0.5f);
  w = m + 0.03125f;
  if (i & 1) {
    typedef _Float16 h2 __attribute__((ext_vector_type(2)));
    typedef float f2 __attribute__((ext_vector_type(2)));
    const f2 pair = {e, f};
    const h2 packed = __builtin_convertvector(pair, h2);
    u = (float)packed[0] * 0.5f + 0.25f;
  } else {
    u = e * 0.5f + 0.25f;
  }
}

// operands: [16][256] 128-bit register images (8 A slots and 8 B slots interleaved)
template <int DT, int MODE>
__global__ __launch_bounds__(256) void mfma_stream_kernel(const u32x4* __restrict__ operands,
                                                          float* __restrict__ sink, int iters) {
  __shared__ u32x4 lds[8 * 256];
  const int tid = threadIdx.x;
  u32x4 a[8], b[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    a[i] = operands[(size_t)(2 * i) * 256 + tid];
    b[i] = operands[(size_t)(2 * i + 1) * 256 + tid];
    lds[i * 256 + tid] = a[i];
  }
  __syncthreads();
  f32x16 c0, c1, c2, c3;
#pragma unroll
  for (int r = 0; r < 16; ++r) c0[r] = c1[r] = c2[r] = c3[r] = 0.0f;
  float x[8];   // state of the vector filler of mode 2: values that stay in (0, 1]
#pragma unroll
  for (int r = 0; r < 8; ++r) x[r] = 0.5f + 0.001f * (float)((tid + r) & 63);
  if constexpr (MODE == 0) {
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        c0 = mfma<DT>(a[i], b[i], c0);
        c1 = mfma<DT>(a[(i + 1) & 7], b[i], c1);
        c2 = mfma<DT>(a[i], b[(i + 3) & 7], c2);
        c3 = mfma<DT>(a[(i + 5) & 7], b[(i + 2) & 7], c3);
      }
    }
  } else if constexpr (MODE == 1 || MODE == 2) {
    // volatile: the reads are loop-invariant and would otherwise be hoisted out of the loop.
    // Operands are requested two MFMA groups (8 reads, ~256 cycles of matrix work) ahead of
    // their use, so that the LDS round trip never shows and what is measured is the pipe.
    VolatileLdsU32x4* slot = (VolatileLdsU32x4*)lds + tid;
    u32x4 a0 = slot[0 * 256], a1 = slot[1 * 256], a2 = slot[2 * 256], a3 = slot[5 * 256];
    u32x4 m0 = slot[1 * 256], m1 = slot[2 * 256], m2 = slot[3 * 256], m3 = slot[6 * 256];
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int n = (i + 2) & 7;
        const u32x4 n0 = slot[n * 256], n1 = slot[((n + 1) & 7) * 256], n2 = slot[((n + 2) & 7) * 256],
                    n3 = slot[((n + 5) & 7) * 256];
        // the scheduler would otherwise sink every read to just before its use, with a full
        // wait for it ahead of each MFMA
        __builtin_amdgcn_sched_barrier(0);
        c0 = mfma<DT>(a0, b[i], c0);
        if constexpr (MODE == 2) vector_work(x, i);
        c1 = mfma<DT>(a1, b[i], c1);
        if constexpr (MODE == 2) vector_work(x, i + 1);
        c2 = mfma<DT>(a2, b[(i + 3) & 7], c2);
        if constexpr (MODE == 2) vector_work(x, i + 2);
        c3 = mfma<DT>(a3, b[(i + 2) & 7], c3);
        if constexpr (MODE == 2) vector_work(x, i + 3);
        a0 = m0;
        a1 = m1;
        a2 = m2;
        a3 = m3;
        m0 = n0;
        m1 = n1;
        m2 = n2;
        m3 = n3;
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  }
  float s = 0.0f;
#pragma unroll
  for (int r = 0; r < 16; ++r) s += c0[r] + c1[r] + c2[r] + c3[r];
#pragma unroll
  for (int r = 0; r < 8; ++r) s += x[r];
  sink[(size_t)blockIdx.x * 256 + tid] = s;
}

}  // namespace

extern "C" int ellm_diag_mfma_stream(int mode, int dtype, const void* operands, float* sink,
                                     int workgroups, int iters, void* stream, double* flops) {
  if (!operands || !sink || workgroups <= 0 || iters <= 0 || (mode < 0 || mode > 2) ||
      (dtype != 0 && dtype != 1))
    return 1;
  if (mode == 2) {
    if (dtype == 0) hipLaunchKernelGGL((mfma_stream_kernel<0, 2>), dim3((uint32_t)workgroups), dim3(256), 0, (hipStream_t)stream, (const u32x4*)operands, sink, iters);
    else hipLaunchKernelGGL((mfma_stream_kernel<1, 2>), dim3((uint32_t)workgroups), dim3(256), 0, (hipStream_t)stream, (const u32x4*)operands, sink, iters);
    if (hipGetLastError() != hipSuccess) return 4;
    if (flops) *flops = (double)workgroups * 4.0 * (double)iters * 32.0 * 32768.0;
    return 0;
  }
  const dim3 grid((uint32_t)workgroups), block(256);
  const u32x4* ops = (const u32x4*)operands;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == 0 && mode == 0) hipLaunchKernelGGL((mfma_stream_kernel<0, 0>), grid, block, 0, s, ops, sink, iters);
  if (dtype == 0 && mode == 1) hipLaunchKernelGGL((mfma_stream_kernel<0, 1>), grid, block, 0, s, ops, sink, iters);
  if (dtype == 1 && mode == 0) hipLaunchKernelGGL((mfma_stream_kernel<1, 0>), grid, block, 0, s, ops, sink, iters);
  if (dtype == 1 && mode == 1) hipLaunchKernelGGL((mfma_stream_kernel<1, 1>), grid, block, 0, s, ops, sink, iters);
  if (hipGetLastError() != hipSuccess) return 4;
  // 4 waves a workgroup x iters x 32 MFMAs x (32 x 32 x 16 multiply-adds = 32768 flop)
  if (flops) *flops = (double)workgroups * 4.0 * (double)iters * 32.0 * 32768.0;
  return 0;
}
