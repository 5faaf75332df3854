// Projections for a few token rows (a single-token step over up to 64 sequences): the
// weights are read exactly once and the kernel is bound by that stream (HBM), not by
// MFMA.  Same arithmetic and epilogue as the tile kernel of project.hip.
//
// A workgroup owns one head (128 output columns) and one slice of K (256 or 64
// elements); its four waves take 32 columns each.  A lane fetches its MFMA operands
// straight from memory in operand layout (16x16x32: row = lane % 16, eight consecutive
// K elements at 8 * (lane / 16)): every weight byte is fetched by exactly one lane of one
// wave, all fetches of a wave are issued before the first is used, and nothing goes
// through LDS.  The product is computed transposed (weights = A operand, token rows = B
// operand), so a lane's accumulator holds four consecutive columns of one token.
// The K slices of a head are added up by the last workgroup of the head to arrive (an
// arrival counter per head that resets itself; partial sums in a workspace, written and
// read with device-coherent accesses), in slice order, so the result does not depend on
// the order of arrival; that workgroup then normalises, rotates, adds the residual and
// stores the head's rows.
#include "project_common.hpp"

namespace ellm {
using namespace proj;
namespace {

constexpr int kSmallThreads = 256;
constexpr int kFoldMax = 16;  // K slices summed per pass of the final fold

// Device-coherent 16-byte store (the compiler has no 16-byte atomic store).  The wait
// states after it are what the hardware needs between a store of more than 8 bytes and
// the next write to its data registers; the compiler adds them after its own stores and
// cannot see that this statement is one.
__device__ __forceinline__ void store_coherent128(float* p, f32x4 v) {
  asm volatile("global_store_dwordx4 %0, %1, off sc1\n\ts_nop 1" ::"v"(p), "v"(v) : "memory");
}
__device__ __forceinline__ f32x4 load_coherent128_nowait(const float* p) {
  f32x4 v;
  asm volatile("global_load_dwordx4 %0, %1, off sc1" : "=v"(v) : "v"(p) : "memory");
  return v;
}
__device__ __forceinline__ void wait_vm_done() { __builtin_amdgcn_s_waitcnt(0x0F70); }

// NTB: 16-token blocks (1, 2 or 4); STEPS: 32-element K steps per slice (8 or 2).
template <typename S, int MODE, int NTB, int STEPS>
__global__ __launch_bounds__(kSmallThreads) void project_small_kernel(ProjectKernelArgs p, float* ws,
                                                                      uint32_t* counters,
                                                                      uint32_t ksplit) {
  using M = Mfma<S>;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int i16 = lane & 15, q4 = lane >> 4;
  const uint32_t hh = blockIdx.x / ksplit, ks = blockIdx.x % ksplit;
  const uint32_t K = p.K;
  const uint32_t k0 = ks * (32 * STEPS);
  const uint32_t seg = (hh < p.heads0) ? 0u : (hh < p.heads0 + p.heads_kv ? 1u : 2u);
  const uint32_t hs = hh - (seg == 0 ? 0u : (seg == 1 ? p.heads0 : p.heads0 + p.heads_kv));
  constexpr int kRowsCap = 16 * NTB;

  // operand fetches: weights rows hs * 128 + 32 wave + 16 nb + i16, token rows 16 tb + i16
  const uint16_t* wbase = p.w[seg] + ((size_t)hs * kHeadDim + 32 * wave + i16) * K + k0 + 8 * q4;
  u32x4 wreg[2][STEPS];
#pragma unroll
  for (int nb = 0; nb < 2; ++nb)
#pragma unroll
    for (int s = 0; s < STEPS; ++s)
      wreg[nb][s] = __builtin_nontemporal_load((const u32x4*)(wbase + (size_t)16 * nb * K + 32 * s));
  const __amdgpu_buffer_rsrc_t x_rsrc =
      __builtin_amdgcn_make_buffer_rsrc((void*)uniform64(p.x), 0, p.rows * K * 2, kBufFlags);
  u32x4 xreg[NTB][STEPS];  // rows past the last one read as zero
#pragma unroll
  for (int tb = 0; tb < NTB; ++tb)
#pragma unroll
    for (int s = 0; s < STEPS; ++s)
      xreg[tb][s] = __builtin_amdgcn_raw_buffer_load_b128(
          x_rsrc, ((16 * tb + i16) * K + k0 + 8 * q4 + 32 * s) * 2, 0, 0);

  f32x4 acc[2][NTB];
#pragma unroll
  for (int nb = 0; nb < 2; ++nb)
#pragma unroll
    for (int tb = 0; tb < NTB; ++tb) acc[nb][tb] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
  for (int s = 0; s < STEPS; ++s)
#pragma unroll
    for (int nb = 0; nb < 2; ++nb)
#pragma unroll
      for (int tb = 0; tb < NTB; ++tb)
        acc[nb][tb] = M::m16x16x32(wreg[nb][s], xreg[tb][s], acc[nb][tb]);

  // partial sums: [head][slice][token][128 columns]; lane (token i16, columns 4 q4..) of block nb
  float* part = ws + ((size_t)hh * ksplit + ks) * kRowsCap * kHeadDim;
#pragma unroll
  for (int nb = 0; nb < 2; ++nb)
#pragma unroll
    for (int tb = 0; tb < NTB; ++tb)
      store_coherent128(part + (size_t)(16 * tb + i16) * kHeadDim + 32 * wave + 16 * nb + 4 * q4,
                        acc[nb][tb]);

  // arrival: every thread's stores acknowledged, then one count per workgroup
  __shared__ uint32_t s_last;
  wait_vm_done();
  __syncthreads();
  if (tid == 0) {
    uint32_t* c = counters + hh;
    const uint32_t old = __hip_atomic_fetch_add(c, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const uint32_t last = (old + 1 == ksplit) ? 1u : 0u;
    if (last) __hip_atomic_store(c, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // for the next launch
    s_last = last;
  }
  __syncthreads();
  if (s_last == 0) return;

  // ---- the head's last workgroup: fold the slices, finish the rows ------------------
  // thread -> token tid / 16 (+ 16 per pass), columns 8 c .. 8 c + 7 with c = tid % 16
  const bool finalize = MODE == kModeQkv && ((seg == 1) || (seg == 0 && p.finalize0));
  uint16_t* const dst = (seg == 0) ? p.out0 : (seg == 1 ? p.k_out : p.v_out);
  const int c8 = tid & 15;
  const float* head_parts = ws + (size_t)hh * ksplit * kRowsCap * kHeadDim;
  for (int pass = 0; pass < NTB; ++pass) {
    const uint32_t R = 16 * pass + (tid >> 4);
    f32x4 lo = {0.0f, 0.0f, 0.0f, 0.0f}, hi = {0.0f, 0.0f, 0.0f, 0.0f};
    for (uint32_t first = 0; first < ksplit; first += kFoldMax) {
      f32x4 a[kFoldMax], b[kFoldMax];
#pragma unroll
      for (int i = 0; i < kFoldMax; ++i) {
        if (first + i < ksplit) {
          const float* src = head_parts + ((size_t)(first + i) * kRowsCap + R) * kHeadDim + 8 * c8;
          a[i] = load_coherent128_nowait(src);
          b[i] = load_coherent128_nowait(src + 4);
        }
      }
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
      for (int i = 0; i < kFoldMax; ++i) {
        asm volatile("" : "+v"(a[i]), "+v"(b[i]));  // nothing reads them ahead of the wait
        if (first + i < ksplit) {
          lo += a[i];
          hi += b[i];
        }
      }
    }
    const uint32_t t = R / p.batch_pitch, b = R % p.batch_pitch;
    const bool live = R < p.rows && b < p.batch;
    uint32_t pos = t;
    if (p.positions)
      pos += live ? min(p.positions[b], p.max_start) : 0u;
    else
      pos += p.position_index;
    float o[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    if (MODE == kModeQkv) {
      float ss = 0.0f;
#pragma unroll
      for (int e = 0; e < 8; ++e) ss = fmaf(o[e], o[e], ss);
#pragma unroll
      for (int m = 1; m < 16; m <<= 1) ss += __shfl_xor(ss, m, 16);
      const float inv = finalize ? 1.0f / (sqrtf(ss / (float)kHeadDim) + p.eps) : 1.0f;
      const uint32_t one_zero = M::pack2(1.0f, 0.0f);
      u32x4 rr = {one_zero, one_zero, one_zero, one_zero};
      if (finalize && live)
        rr = load16(p.rope + (size_t)pos * p.rope_pos_stride + (size_t)hs * p.rope_head_stride + 8 * c8);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float cs = M::to_float((uint16_t)(rr[e] & 0xffffu)), sn = M::to_float((uint16_t)(rr[e] >> 16));
        const float y0 = o[2 * e] * inv, y1 = o[2 * e + 1] * inv;
        o[2 * e] = y0 * cs - y1 * sn;
        o[2 * e + 1] = y0 * sn + y1 * cs;
      }
    }
    if (live) {
      size_t off;
      if (seg == 0)
        off = (size_t)R * p.ld0 + hs * kHeadDim + 8 * c8;
      else
        off = (size_t)b * p.kv_stride_seq + (size_t)hs * p.kv_stride_head + (size_t)pos * p.kv_stride_pos +
              8 * c8;
      if (MODE == kModeAdd) {
        const u32x4 rs = load16(p.residual + off);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          o[2 * e] += M::to_float((uint16_t)(rs[e] & 0xffffu));
          o[2 * e + 1] += M::to_float((uint16_t)(rs[e] >> 16));
        }
      }
      const u32x4 packed = {M::pack2(o[0], o[1]), M::pack2(o[2], o[3]), M::pack2(o[4], o[5]),
                            M::pack2(o[6], o[7])};
      store16(dst + off, packed);
    }
  }
}

template <typename S, int MODE, int NTB>
hipError_t launch_steps(const ProjectKernelArgs& p, float* ws, uint32_t* counters, uint32_t heads,
                        hipStream_t stream) {
  if (p.K % 256 == 0) {
    const uint32_t ksplit = p.K / 256;
    hipLaunchKernelGGL((project_small_kernel<S, MODE, NTB, 8>), dim3(heads * ksplit), dim3(kSmallThreads),
                       0, stream, p, ws, counters, ksplit);
  } else {
    const uint32_t ksplit = p.K / 64;
    hipLaunchKernelGGL((project_small_kernel<S, MODE, NTB, 2>), dim3(heads * ksplit), dim3(kSmallThreads),
                       0, stream, p, ws, counters, ksplit);
  }
  return hipGetLastError();
}

template <typename S, int MODE>
hipError_t launch_blocks(const ProjectKernelArgs& p, float* ws, uint32_t* counters, uint32_t heads,
                         hipStream_t stream) {
  if (p.rows <= 16) return launch_steps<S, MODE, 1>(p, ws, counters, heads, stream);
  if (p.rows <= 32) return launch_steps<S, MODE, 2>(p, ws, counters, heads, stream);
  return launch_steps<S, MODE, 4>(p, ws, counters, heads, stream);
}

}  // namespace

namespace proj {

// Workspace of the streaming kernel for `heads` heads and K columns: partial sums
// [head][slice][64][128] floats; one counter per head.
size_t small_workspace_floats(uint32_t heads, uint32_t K) {
  const uint32_t ksplit = (K % 256 == 0) ? K / 256 : K / 64;
  return (size_t)heads * ksplit * kSmallRowsMax * kHeadDim;
}

hipError_t launch_project_small(const ProjectKernelArgs& p, float* ws, uint32_t* counters, int dtype,
                                bool add, hipStream_t stream) {
  const uint32_t heads = p.heads0 + 2 * p.heads_kv;
  if (add)
    return dtype == 0 ? launch_blocks<F16, kModeAdd>(p, ws, counters, heads, stream)
                      : launch_blocks<BF16, kModeAdd>(p, ws, counters, heads, stream);
  return dtype == 0 ? launch_blocks<F16, kModeQkv>(p, ws, counters, heads, stream)
                    : launch_blocks<BF16, kModeQkv>(p, ws, counters, heads, stream);
}

}  // namespace proj
}  // namespace ellm
