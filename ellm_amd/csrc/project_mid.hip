// Projection tile kernel for a few hundred to a few thousand rows, where the 256 x 256
// tiles of project.hip leave most compute units without a workgroup (1536 rows, the
// reference's own serving shape of 64 positions x 24 sequences, src/serving/start copy.rs:30,
// make 6 x 20 of them for the fused Q/K/V projection and 6 x 8 for the output projection).
// Same formulation (C^T = W . X^T on v_mfma_f32_32x32x16, a lane owns a token), same LDS
// layout and the same epilogue; the tile is 128 tokens x one head, two workgroups fit a
// compute unit (the second one fills the gaps a short loop leaves).
#include "project_epilogue.hpp"

namespace ellm {
namespace proj {
namespace {

constexpr int kMidTokens = 128;                   // tokens per workgroup; output columns: one head
constexpr int kMidKc = 64;                        // K elements per chunk: one 128-byte line per row
constexpr int kMidRowPitch = kMidKc * 2;          // unpadded; pieces permuted as in project.hip
constexpr int kMidStageBytes = (kMidTokens + kHeadDim) * kMidRowPitch;  // X rows then W rows
constexpr int kMidLdsBytes = 2 * kMidStageBytes;
constexpr int kMidThreads = 256;
static_assert(4 * kEpWaveBytes <= kMidLdsBytes, "the epilogue reuses the stages");

template <typename S, int MODE>
__global__ __launch_bounds__(kMidThreads, 2) void project_mid_kernel(ProjectKernelArgs p) {
  using M = Mfma<S>;
  extern __shared__ __attribute__((aligned(16))) uint8_t mid_smem[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int j = lane & 31, g = lane >> 5;

  // workgroup -> tile: ids that share id % 8 (one XCD, one L2) are made consecutive; a
  // head's token tiles are neighbours, so a head's weights are fetched by one L2 only
  uint32_t tm, tn;
  {
    const uint32_t total = p.tiles_m * p.tiles_n;
    const uint32_t q = total >> 3, r = total & 7, xcd = blockIdx.x & 7, idx = blockIdx.x >> 3;
    const uint32_t pid = xcd * q + min(xcd, r) + idx;
    tn = pid / p.tiles_m;
    tm = pid % p.tiles_m;
  }
  const uint32_t K = p.K;
  const uint32_t n_chunks = K / kMidKc;
  const uint32_t row0 = tm * kMidTokens;
  const uint32_t rows_here = min(p.rows - row0, (uint32_t)kMidTokens);
  const __amdgpu_buffer_rsrc_t x_rsrc = __builtin_amdgcn_make_buffer_rsrc(
      (void*)(uniform64(p.x) + (uint64_t)row0 * K * 2), 0, rows_here * K * 2, kBufFlags);
  const uint16_t* wbase = p.w[0];
  uint32_t hs = tn;
  if (tn >= p.heads0 + p.heads_kv) {
    wbase = p.w[2];
    hs = tn - p.heads0 - p.heads_kv;
  } else if (tn >= p.heads0) {
    wbase = p.w[1];
    hs = tn - p.heads0;
  }
  const __amdgpu_buffer_rsrc_t w_rsrc = __builtin_amdgcn_make_buffer_rsrc(
      (void*)(uniform64(wbase) + (uint64_t)hs * kHeadDim * K * 2), 0, kHeadDim * K * 2, kBufFlags);

  // staging: thread -> row tid / 8 (+ 32 i) of the 128 X rows (i < 4) or the 128 W rows,
  // 16-byte piece tid % 8 of the chunk's 128 bytes: eight lanes fetch one whole cache line
  const uint32_t st_row = tid >> 3, st_piece = tid & 7;
  const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)mid_smem;
  const uint32_t st_store = lds0 + st_row * kMidRowPitch + ((st_piece ^ ((st_row >> 1) & 7)) * 16);
  u32x4 stg[8];
  // (a chunk past the last one fetches bytes of the next row, or zeros past the end of the
  // buffer, into a stage nobody reads)
  auto load_chunk = [&](uint32_t chunk) {
    const uint32_t soff = chunk * (kMidKc * 2);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const uint32_t off = (st_row + 32 * (i & 3)) * K * 2 + st_piece * 16;
      stg[i] = __builtin_amdgcn_raw_buffer_load_b128(i < 4 ? x_rsrc : w_rsrc, off, soff, 0);
    }
  };
  auto store_chunk = [&](uint32_t stage) {
#pragma unroll
    for (int i = 0; i < 8; ++i) *(LdsVec4*)(st_store + stage + 32 * i * kMidRowPitch) = stg[i];
  };

  f32x16 acc[4][1];  // [column block nb][token block]
#pragma unroll
  for (int nb = 0; nb < 4; ++nb)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[nb][0][r] = 0.0f;

  // operand reads: lane (j, g) takes row j of a 32-row block, piece 2 step + g, permuted
  const uint32_t swz = (j >> 1) & 7;
  const uint32_t x_row = lds0 + (wave * 32 + j) * kMidRowPitch;
  const uint32_t w_row = lds0 + (kMidTokens + j) * kMidRowPitch;

  // operands of one 16-wide step: the X block of this wave and the head's four W blocks
  u32x4 ox[2], ow[2][4];
  auto read_operand = [&](auto set_, uint32_t stage, int st, int o) {
    constexpr int set = decltype(set_)::value;
    const uint32_t piece = ((2 * st + g) ^ swz) * 16;
    if (o == 0)
      ox[set] = *(const LdsVec4*)(x_row + stage + piece);
    else
      ow[set][o - 1] = *(const LdsVec4*)(w_row + stage + 32 * (o - 1) * kMidRowPitch + piece);
  };
  auto load_piece = [&](uint32_t chunk, int i) {
    const uint32_t off = (st_row + 32 * (i & 3)) * K * 2 + st_piece * 16;
    stg[i] = __builtin_amdgcn_raw_buffer_load_b128(i < 4 ? x_rsrc : w_rsrc, off, chunk * (kMidKc * 2), 0);
  };

  load_chunk(0);
  store_chunk(0);
  load_chunk(1);
  __syncthreads();
#pragma unroll
  for (int o = 0; o < 5; ++o) read_operand(std::integral_constant<int, 0>{}, 0, 0, o);

  // One iteration = one chunk = four 16-wide steps of four MFMAs.  The operands of a step
  // are read during the step before it, across chunks too; the staging registers (chunk
  // c + 1, requested an iteration earlier) are stored during steps 0-2 and refilled with
  // chunk c + 2 during step 3.  One barrier, after step 2.  It orders both hazards: the
  // stage that this iteration's stores fill (chunk c - 1's) was last read for step 3 of
  // chunk c - 1, and those reads had returned before the previous barrier; and chunk c + 1
  // is complete before the reads of its first step, issued during step 3.
  for (uint32_t c = 0; c < n_chunks; ++c) {
    const uint32_t cur = (c & 1) * kMidStageBytes, nxt = kMidStageBytes - cur;
    __builtin_amdgcn_sched_barrier(0);
    static_for<16>([&](auto n_) {
      constexpr int n = decltype(n_)::value;
      constexpr int st = n >> 2, nb = n & 3;
      constexpr int set = st & 1;
      acc[nb][0] = M::m32x32x16(ow[set][nb], ox[set], acc[nb][0]);
      // five reads for the next step over this step's four MFMAs
      const uint32_t from = (st < 3) ? cur : nxt;
      constexpr int next_st = (st + 1) & 3;
      read_operand(std::integral_constant<int, 1 - set>{}, from, next_st, nb == 0 ? 0 : nb + 1);
      if constexpr (nb == 0) read_operand(std::integral_constant<int, 1 - set>{}, from, next_st, 1);
      if constexpr (st < 3) {
        // eight staging stores over twelve MFMAs
        if constexpr (n % 3 != 2) *(LdsVec4*)(st_store + nxt + 32 * (n - n / 3) * kMidRowPitch) = stg[n - n / 3];
      } else {
        load_piece(c + 2, 2 * nb);
        load_piece(c + 2, 2 * nb + 1);
      }
      if constexpr (n == 11) {
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        __builtin_amdgcn_s_barrier();
      }
      __builtin_amdgcn_sched_barrier(0);
    });
  }
  __syncthreads();
  finish_head<S, MODE, 1>(p, acc, tn, row0 + 32 * wave, lds0 + wave * kEpWaveBytes, lane);
}

}  // namespace

hipError_t mid_prepare() {
  const void* kernels[] = {
      (const void*)project_mid_kernel<F16, kModeQkv>, (const void*)project_mid_kernel<BF16, kModeQkv>,
      (const void*)project_mid_kernel<F16, kModeAdd>, (const void*)project_mid_kernel<BF16, kModeAdd>};
  for (const void* k : kernels) {
    const hipError_t e =
        hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, kMidLdsBytes);
    if (e != hipSuccess) return e;
  }
  return hipSuccess;
}

hipError_t launch_project_mid(ProjectKernelArgs p, int dtype, bool add, hipStream_t stream) {
  p.tiles_m = (p.rows + kMidTokens - 1) / kMidTokens;
  p.tiles_n = p.heads0 + 2 * p.heads_kv;
  const uint32_t blocks = p.tiles_m * p.tiles_n;
  auto go = [&](auto kernel) {
    hipLaunchKernelGGL(kernel, dim3(blocks), dim3(kMidThreads), kMidLdsBytes, stream, p);
    return hipGetLastError();
  };
  if (add) return dtype == 0 ? go(project_mid_kernel<F16, kModeAdd>) : go(project_mid_kernel<BF16, kModeAdd>);
  return dtype == 0 ? go(project_mid_kernel<F16, kModeQkv>) : go(project_mid_kernel<BF16, kModeQkv>);
}

}  // namespace proj
}  // namespace ellm
