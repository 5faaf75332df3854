// Projections for up to 64 token rows (a single-token step over that many sequences, a
// short chunk): the weights are read exactly once and the kernel is bound by that stream
// (HBM), not by MFMA.  Same arithmetic and epilogue as the tile kernel of project.hip.
//
// A workgroup owns 16 or 32 output columns (one or two 16x16x32 MFMA block rows, which
// share the token operand) and all of K: whole weight rows, contiguous in memory, so the
// stream of a workgroup stays inside a few DRAM pages.  Its waves split K, 256 elements a wave and round; a lane fetches its
// MFMA operands straight from memory in operand layout (row = lane % 16, eight
// consecutive K elements at 8 * (lane / 16)), every weight byte is fetched by exactly one
// lane, all fetches of a round are issued before the first is used, nothing of the
// weights goes through LDS.  The product is computed transposed (weights = A operand,
// token rows = B operand), so a lane's accumulator holds four consecutive columns of one
// token.  The waves' sums meet in LDS.
// Columns that are not normalised (value heads, the output projection) are finished by
// their own workgroup.  A normalised head needs the sum of squares over its 128 columns,
// i.e. over four or eight workgroups: each leaves its columns in a workspace (device-coherent
// stores) and counts itself in; the last of them to arrive reads the head back,
// normalises, rotates and stores it.  The counters reset themselves.
#include "project_common.hpp"

namespace ellm {
using namespace proj;
namespace {

constexpr int kStepsPerRound = 8;            // 32-element K steps a wave has in flight: 256 elements
constexpr int kRoundK = 32 * kStepsPerRound;

__device__ __forceinline__ void store_coherent(float* p, float v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// Device-coherent 16-byte load at byte offset `off` of a table: a buffer load with the sc1
// cache-policy bit (what the compiler's own agent-scope atomic loads carry; it has no 16-byte
// atomic load).  As a builtin the compiler tracks the load's completion itself.
constexpr int kCachePolicySc1 = 16;
__device__ __forceinline__ f32x4 load_coherent128(__amdgpu_buffer_rsrc_t table, uint32_t off) {
  return __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(table, off, 0, kCachePolicySc1));
}
__device__ __forceinline__ void wait_vm_done() { __builtin_amdgcn_s_waitcnt(0x0F70); }

typedef __attribute__((address_space(3))) u32x4 LdsVec4;

// NTB: 16-token blocks per pass (1 or 2); NB: 16-column MFMA blocks per workgroup (1 or 2), or 0: half
// a block, 8 columns (the other 8 rows of the MFMA's weight operand are zero), for outputs so narrow
// that 16-column workgroups would leave compute units without one (kModeAdd and kModeRaw only).
// blockDim.x = 64 * waves, waves = min(16, K / 256).  `passes` passes of 16 NTB token rows
// each reuse the weight operands, which stay in registers; more than one pass needs
// waves == K / 256 (one round of K per wave).
// VIA_LDS (waves == K / 256 and the rows fit): the workgroup's weight rows, one contiguous
// region of memory, are fetched in 1 KB pieces (a wave instruction = 1 KB of one row) and
// handed to the MFMA operand layout through LDS; fetching them in operand layout directly
// (16 rows x 64 B an instruction) makes the same stream a third slower.
template <typename S, int MODE, int NTB, int NB, bool VIA_LDS>
__global__ __launch_bounds__((NTB == 2 || NB == 2) ? 512 : 1024) void project_small_kernel(ProjectKernelArgs p, float* ws,
                                                             uint32_t* counters, uint32_t passes) {
  using M = Mfma<S>;
  static_assert(NB != 0 || MODE != kModeQkv, "the heads' finishing step reads whole 16-column blocks");
  constexpr int kColBlocks = NB ? NB : 1, kGroupCols = NB ? 16 * NB : 8, kGroupsPerHead = kHeadDim / kGroupCols;
  constexpr bool kHalf = NB == 0;
  constexpr bool kEarlyResidual = MODE == kModeAdd && kHalf;
  constexpr int kPassRows = 16 * NTB;
  extern __shared__ __attribute__((aligned(16))) float sums[];  // [wave][NTB][16 tokens][kGroupCols]
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, n_waves = blockDim.x >> 6;
  const int i16 = lane & 15, q4 = lane >> 4;
  const uint32_t K = p.K;
  const uint32_t hh = blockIdx.x / kGroupsPerHead, cg = blockIdx.x % kGroupsPerHead;
  const uint32_t seg = (hh < p.heads0) ? 0u : (hh < p.heads0 + p.heads_kv ? 1u : 2u);
  const uint32_t hs = hh - (seg == 0 ? 0u : (seg == 1 ? p.heads0 : p.heads0 + p.heads_kv));
  const uint32_t rows_cap = passes * kPassRows;
  const bool finalize = MODE == kModeQkv && ((seg == 1) || (seg == 0 && p.finalize0));
  uint16_t* const dst = (seg == 0) ? p.out0 : (seg == 1 ? p.k_out : p.v_out);

  const uint16_t* wrow = p.w[seg] + ((size_t)hs * kHeadDim + kGroupCols * cg + (kHalf ? (i16 & 7) : i16)) * K + 8 * q4;
  const size_t wblock = (size_t)16 * K;  // elements between the rows of consecutive column blocks
  const __amdgpu_buffer_rsrc_t x_rsrc =
      __builtin_amdgcn_make_buffer_rsrc((void*)uniform64(p.x), 0, p.rows * K * 2, kBufFlags);
  const uint32_t k_first = wave * kRoundK;
  // token rows of pass `pass`, K slice at k0 (rows past the last read as zero)
  auto fetch_x = [&](u32x4 (&x)[NTB][kStepsPerRound], uint32_t pass, uint32_t k0) {
#pragma unroll
    for (int tb = 0; tb < NTB; ++tb)
#pragma unroll
      for (int s = 0; s < kStepsPerRound; ++s)
        x[tb][s] = __builtin_amdgcn_raw_buffer_load_b128(
            x_rsrc, ((pass * kPassRows + 16 * tb + i16) * K + k0 + 8 * q4 + 32 * s) * 2, 0, 0);
  };
  auto fetch_w = [&](u32x4 (&w)[kColBlocks][kStepsPerRound], uint32_t k0) {
#pragma unroll
    for (int nb = 0; nb < kColBlocks; ++nb)
#pragma unroll
      for (int s = 0; s < kStepsPerRound; ++s)
        w[nb][s] = (kHalf && i16 >= 8) ? u32x4{0, 0, 0, 0}
                                       : __builtin_nontemporal_load((const u32x4*)(wrow + nb * wblock + k0 + 32 * s));
  };

  constexpr int kQuads = kGroupCols / 4;
  // The waves' sums of one pass meet in LDS; threads 0 .. 4 kGroupCols NTB - 1 (token tid / kQuads
  // of the pass, four columns of the group) add them up and either finish the row or leave it
  // for the head's last workgroup.
  auto finish_pass = [&](uint32_t pass, f32x4 (&acc)[kColBlocks][NTB]) {
    // the residual's piece is requested before the sums meet, not behind them (where the
    // registers are there for it: the 16-wave forms run at 128 a lane)
    u32x2 rs = {0u, 0u};
    if constexpr (kEarlyResidual) {
      if (tid < 16 * kQuads * NTB) {
        const uint32_t R = pass * kPassRows + tid / kQuads;
        if (R < p.rows && R % p.batch_pitch < p.batch)
          rs = *(const u32x2*)(p.residual + (size_t)R * p.ld0 + hs * kHeadDim + kGroupCols * cg + 4 * (tid % kQuads));
      }
    }
    // lane (token i16, columns 16 nb + 4 q4 .. + 3)
#pragma unroll
    for (int nb = 0; nb < kColBlocks; ++nb)
#pragma unroll
      for (int tb = 0; tb < NTB; ++tb)
        if (!kHalf || q4 < 2)
          *(f32x4*)(sums + ((wave * NTB + tb) * 16 + i16) * kGroupCols + 16 * nb + 4 * q4) = acc[nb][tb];
    __syncthreads();
    if (tid < 16 * kQuads * NTB) {
      const uint32_t R = pass * kPassRows + tid / kQuads, c4 = tid % kQuads;
      f32x4 v = {0.0f, 0.0f, 0.0f, 0.0f};
      for (int w = 0; w < n_waves; ++w)
        v += *(const f32x4*)(sums + (w * kPassRows + tid / kQuads) * kGroupCols + 4 * c4);
      if constexpr (MODE == kModeRaw) {
        // plain stores: the kernel that reads them is the next launch on the stream
        const uint32_t cols = (p.heads0 + 2 * p.heads_kv) * kHeadDim;
        if (R < p.rows && R % p.batch_pitch < p.batch)
          *(f32x4*)(ws + (size_t)R * cols + hh * kHeadDim + kGroupCols * cg + 4 * c4) = v;
      } else if (finalize) {
        float* to = ws + (((size_t)hh * kGroupsPerHead + cg) * rows_cap + R) * kGroupCols + 4 * c4;
#pragma unroll
        for (int e = 0; e < 4; ++e) store_coherent(to + e, v[e]);
      } else {
        const uint32_t t = R / p.batch_pitch, b = R % p.batch_pitch;
        if (R < p.rows && b < p.batch) {
          size_t off;
          if (seg == 0) {
            off = (size_t)R * p.ld0 + hs * kHeadDim + kGroupCols * cg + 4 * c4;
          } else {
            const uint32_t pos = t + (p.positions ? min(p.positions[b], p.max_start) : p.position_index);
            off = kv_row_offset(p, b, hs, pos) + kGroupCols * cg + 4 * c4;
          }
          if (MODE == kModeAdd) {
            if constexpr (!kEarlyResidual) rs = *(const u32x2*)(p.residual + off);
            v[0] += M::to_float((uint16_t)(rs[0] & 0xffffu));
            v[1] += M::to_float((uint16_t)(rs[0] >> 16));
            v[2] += M::to_float((uint16_t)(rs[1] & 0xffffu));
            v[3] += M::to_float((uint16_t)(rs[1] >> 16));
          }
          const u32x2 packed = {M::pack2(v[0], v[1]), M::pack2(v[2], v[3])};
          *(u32x2*)(dst + off) = packed;
        }
      }
    }
  };

  if constexpr (VIA_LDS) {
    u32x4 wreg[kColBlocks][kStepsPerRound], xcur[NTB][kStepsPerRound];
    {
      const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) float*)sums;
      const uint8_t* wg_rows = (const uint8_t*)(p.w[seg] + ((size_t)hs * kHeadDim + kGroupCols * cg) * K);
      const uint32_t row_bytes = 2 * K, pitch = row_bytes + 16;  // + 16: the 16 rows of an operand read tile the banks
      constexpr int kPieces = kGroupCols / 2;                    // 1 KB pieces per wave (waves x 256 = K)
      u32x4 stg[kPieces];
#pragma unroll
      for (int u = 0; u < kPieces; ++u)
        stg[u] = __builtin_nontemporal_load((const u32x4*)(wg_rows + (size_t)(wave * kPieces + u) * 1024 + lane * 16));
      fetch_x(xcur, 0, k_first);
      __builtin_amdgcn_sched_barrier(0);  // every fetch is on its way before the first use
#pragma unroll
      for (int u = 0; u < kPieces; ++u) {
        const uint32_t off = (wave * kPieces + u) * 1024 + lane * 16;
        const uint32_t row = off / row_bytes;
        *(LdsVec4*)(lds0 + row * pitch + (off - row * row_bytes)) = stg[u];
      }
      __syncthreads();
#pragma unroll
      for (int nb = 0; nb < kColBlocks; ++nb)
#pragma unroll
        for (int s = 0; s < kStepsPerRound; ++s)
          wreg[nb][s] = (kHalf && i16 >= 8)
                            ? u32x4{0, 0, 0, 0}
                            : (u32x4)*(const LdsVec4*)(lds0 + (16 * nb + i16) * pitch + (k_first + 32 * s + 8 * q4) * 2);
      __syncthreads();  // the sums reuse the rows' LDS
    }
    // the weight operands stay in registers; the token rows of the next pass are requested
    // before those of this one are used, where the registers are there for them (a second set
    // of token rows in the widest forms would not fit, and a kernel that spills, by however
    // little, pays several microseconds a launch for its scratch memory to be set up)
    constexpr bool kAhead = NTB == 1 && !(MODE == kModeQkv && NB == 1) && !kEarlyResidual;
    for (uint32_t pass = 0; pass < passes; ++pass) {
      u32x4 xnext[kAhead ? NTB : 1][kAhead ? kStepsPerRound : 1];
      const bool more = pass + 1 < passes;  // (uniform)
      if constexpr (kAhead) {
        if (more) fetch_x(xnext, pass + 1, k_first);
      }
      f32x4 acc[kColBlocks][NTB];
#pragma unroll
      for (int nb = 0; nb < kColBlocks; ++nb)
#pragma unroll
        for (int tb = 0; tb < NTB; ++tb) acc[nb][tb] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
      for (int s = 0; s < kStepsPerRound; ++s)
#pragma unroll
        for (int nb = 0; nb < kColBlocks; ++nb)
#pragma unroll
          for (int tb = 0; tb < NTB; ++tb) acc[nb][tb] = M::m16x16x32(wreg[nb][s], xcur[tb][s], acc[nb][tb]);
      if constexpr (!kAhead) {
        if (more) fetch_x(xcur, pass + 1, k_first);
      }
      finish_pass(pass, acc);
      if (more) {
        __syncthreads();  // the sums are rewritten by the next pass
        if constexpr (kAhead) {
#pragma unroll
          for (int tb = 0; tb < NTB; ++tb)
#pragma unroll
            for (int s = 0; s < kStepsPerRound; ++s) xcur[tb][s] = xnext[tb][s];
        }
      }
    }
  } else {
    // one pass; a wave walks its rounds of K, operands fetched in MFMA layout
    f32x4 acc[kColBlocks][NTB];
#pragma unroll
    for (int nb = 0; nb < kColBlocks; ++nb)
#pragma unroll
      for (int tb = 0; tb < NTB; ++tb) acc[nb][tb] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    for (uint32_t k0 = k_first; k0 < K; k0 += n_waves * kRoundK) {
      u32x4 wreg[kColBlocks][kStepsPerRound], xreg[NTB][kStepsPerRound];
      fetch_w(wreg, k0);
      fetch_x(xreg, 0, k0);
      __builtin_amdgcn_sched_barrier(0);  // every fetch of the round is on its way before the first use
#pragma unroll
      for (int s = 0; s < kStepsPerRound; ++s)
#pragma unroll
        for (int nb = 0; nb < kColBlocks; ++nb)
#pragma unroll
          for (int tb = 0; tb < NTB; ++tb) acc[nb][tb] = M::m16x16x32(wreg[nb][s], xreg[tb][s], acc[nb][tb]);
    }
    finish_pass(0, acc);
  }
  if (!finalize) return;  // (uniform over the workgroup)

  // arrival: every thread's stores acknowledged, then one count per workgroup
  __shared__ uint32_t s_last;
  wait_vm_done();
  __syncthreads();
  if (tid == 0) {
    uint32_t* c = counters + hh;
    const uint32_t old = __hip_atomic_fetch_add(c, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const uint32_t last = (old + 1 == (uint32_t)kGroupsPerHead) ? 1u : 0u;
    if (last) __hip_atomic_store(c, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // for the next launch
    s_last = last;
  }
  __syncthreads();
  if (s_last == 0) return;

  // ---- the head's last workgroup: thread -> token tid / 16 (+ blockDim / 16 a turn), columns 8 c .. 8 c + 7
  const int c8 = tid & 15;
  constexpr int kOctets = kGroupCols / 8;
  const uint32_t one_zero = M::pack2(1.0f, 0.0f);
  // (the workspace of a handle stays far below 4 GB: byte offsets fit 32 bits)
  const __amdgpu_buffer_rsrc_t ws_rsrc =
      __builtin_amdgcn_make_buffer_rsrc((void*)uniform64(ws), 0, 0xffffffffu, kBufFlags);
  for (uint32_t R = tid >> 4; R < rows_cap; R += blockDim.x >> 4) {
    const uint32_t src = (uint32_t)(
        ((((size_t)hh * kGroupsPerHead + c8 / kOctets) * rows_cap + R) * kGroupCols + 8 * (c8 % kOctets)) * 4);
    const f32x4 lo = load_coherent128(ws_rsrc, src), hi = load_coherent128(ws_rsrc, src + 16);
    const uint32_t t = R / p.batch_pitch, b = R % p.batch_pitch;
    const bool live = R < p.rows && b < p.batch;
    const uint32_t pos = t + (p.positions ? (live ? min(p.positions[b], p.max_start) : 0u) : p.position_index);
    u32x4 rr = {one_zero, one_zero, one_zero, one_zero};
    if (live) rr = load16(p.rope + (size_t)pos * p.rope_pos_stride + (size_t)hs * p.rope_head_stride + 8 * c8);
    const float o[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    float ss = squares8(o);
#pragma unroll
    for (int m = 1; m < 16; m <<= 1) ss += __shfl_xor(ss, m, 16);
    const u32x4 packed = scale_rotate_pack8<S>(o, inverse_rms(ss, p.eps), rr);
    if (live) {
      size_t off;
      if (seg == 0)
        off = (size_t)R * p.ld0 + hs * kHeadDim + 8 * c8;
      else
        off = kv_row_offset(p, b, hs, pos) + 8 * c8;
      store16(dst + off, packed);
    }
  }
}

// Two column blocks a workgroup halve the re-reads of the token rows (every workgroup
// reads all of them) but also the number of workgroups; one compute unit streams at most
// ~55 GB/s, so narrow outputs keep one block to have enough of them.
constexpr uint32_t kLdsBudget = 150 * 1024;

template <typename S, int MODE, int NTB, int NB>
hipError_t launch_one(const ProjectKernelArgs& p, float* ws, uint32_t* counters, uint32_t heads, uint32_t waves,
                      hipStream_t stream) {
  constexpr uint32_t kCols = NB ? 16 * NB : 8;
  const dim3 grid(heads * (kHeadDim / kCols)), block(64 * waves);
  const uint32_t passes = (p.rows + 16 * NTB - 1) / (16 * NTB);
  const uint32_t sums_bytes = waves * NTB * 64 * kCols;
  const uint32_t rows_bytes = kCols * (2 * p.K + 16);
  if (waves * kRoundK == p.K && rows_bytes <= kLdsBudget) {
    const uint32_t lds = rows_bytes > sums_bytes ? rows_bytes : sums_bytes;
    hipLaunchKernelGGL((project_small_kernel<S, MODE, NTB, NB, true>), grid, block, lds, stream, p, ws, counters,
                       passes);
  } else {
    if (passes > 1) return hipErrorInvalidValue;  // (small_kernel_takes keeps such calls away)
    hipLaunchKernelGGL((project_small_kernel<S, MODE, NTB, NB, false>), grid, block, sums_bytes, stream, p, ws,
                       counters, passes);
  }
  return hipGetLastError();
}

template <typename S, int MODE>
hipError_t launch_blocks(const ProjectKernelArgs& p, float* ws, uint32_t* counters, uint32_t heads,
                         hipStream_t stream) {
  uint32_t waves = p.K / kRoundK;
  if (waves > 16) waves = 16;
  // two column blocks: enough columns for >= 128 workgroups, and (where the rows go through LDS) room for 32 rows
  const bool wide = heads * kHeadDim >= 4096 && waves <= 8 &&
                    (waves * kRoundK != p.K || 32 * (2 * p.K + 16) <= kLdsBudget);
  // two token blocks a pass want 512 threads for the finishing step and 256 registers a lane
  const bool two_blocks = p.rows > 16 && waves == 8;
  // 16-column workgroups fewer than three quarters of a 256-unit part: 8 columns each (the output
  // projection 4096 -> 2048: 256 workgroups instead of 128; 7.6 -> us at one row)
  if constexpr (MODE != kModeQkv) {
    if (heads * (kHeadDim / 16) <= 192 && waves * kRoundK == p.K)
      return two_blocks ? launch_one<S, MODE, 2, 0>(p, ws, counters, heads, waves, stream)
                        : launch_one<S, MODE, 1, 0>(p, ws, counters, heads, waves, stream);
  }
  if (!two_blocks)
    return wide ? launch_one<S, MODE, 1, 2>(p, ws, counters, heads, waves, stream)
                : launch_one<S, MODE, 1, 1>(p, ws, counters, heads, waves, stream);
  return wide ? launch_one<S, MODE, 2, 2>(p, ws, counters, heads, waves, stream)
              : launch_one<S, MODE, 2, 1>(p, ws, counters, heads, waves, stream);
}

}  // namespace

namespace proj {

template <typename S, int MODE>
static hipError_t prepare_mode() {
  const void* kernels[] = {(const void*)project_small_kernel<S, MODE, 1, 1, true>,
                           (const void*)project_small_kernel<S, MODE, 1, 2, true>,
                           (const void*)project_small_kernel<S, MODE, 2, 1, true>,
                           (const void*)project_small_kernel<S, MODE, 2, 2, true>};
  for (const void* k : kernels) {
    const hipError_t e = hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBudget);
    if (e != hipSuccess) return e;
  }
  if constexpr (MODE != kModeQkv) {
    const void* narrow[] = {(const void*)project_small_kernel<S, MODE, 1, 0, true>,
                            (const void*)project_small_kernel<S, MODE, 2, 0, true>};
    for (const void* k : narrow) {
      const hipError_t e = hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBudget);
      if (e != hipSuccess) return e;
    }
  }
  return hipSuccess;
}

hipError_t small_prepare() {
  hipError_t e = prepare_mode<F16, kModeQkv>();
  if (e == hipSuccess) e = prepare_mode<BF16, kModeQkv>();
  if (e == hipSuccess) e = prepare_mode<F16, kModeAdd>();
  if (e == hipSuccess) e = prepare_mode<BF16, kModeAdd>();
  if (e == hipSuccess) e = prepare_mode<F16, kModeRaw>();
  if (e == hipSuccess) e = prepare_mode<BF16, kModeRaw>();
  return e;
}

bool small_kernel_takes(uint32_t rows, uint32_t K) {
  if (K % kRoundK != 0 || rows > kSmallRowsMax) return false;
  const uint32_t waves = K / kRoundK;
  if (waves < 4) return false;  // the finishing steps want 256 threads
  if (rows <= 16) return true;
  // several passes (or two token blocks): one round of K per wave, rows through LDS
  return waves <= 16 && 16 * (2 * K + 16) <= kLdsBudget;
}

// Workspace of the streaming kernel: the normalised heads' sums, [head][rows][128] floats
// (rows rounded up to a pass); one counter per head.
size_t small_workspace_floats(uint32_t heads, uint32_t K) {
  (void)K;
  // (also holds the raw rows of a fused single-token step: up to two partial sums of kSmallRowsMax rows)
  return (size_t)heads * (2 * kSmallRowsMax + 32) * kHeadDim;
}

hipError_t launch_project_small(const ProjectKernelArgs& p, float* ws, uint32_t* counters, int dtype,
                                int mode, hipStream_t stream) {
  const uint32_t heads = p.heads0 + 2 * p.heads_kv;
  if (mode == kModeAdd)
    return dtype == 0 ? launch_blocks<F16, kModeAdd>(p, ws, counters, heads, stream)
                      : launch_blocks<BF16, kModeAdd>(p, ws, counters, heads, stream);
  if (mode == kModeRaw)
    return dtype == 0 ? launch_blocks<F16, kModeRaw>(p, ws, counters, heads, stream)
                      : launch_blocks<BF16, kModeRaw>(p, ws, counters, heads, stream);
  return dtype == 0 ? launch_blocks<F16, kModeQkv>(p, ws, counters, heads, stream)
                    : launch_blocks<BF16, kModeQkv>(p, ws, counters, heads, stream);
}

}  // namespace proj
}  // namespace ellm
