// Projection tile kernel for a few hundred to a few thousand rows, where the 256 x 256
// tiles of project.hip leave most compute units without a workgroup (1536 rows, the
// reference's own serving shape of 64 positions x 24 sequences, src/serving/start copy.rs:30,
// make 6 x 20 of them for the fused Q/K/V projection and 6 x 8 for the output projection).
// Same formulation (C^T = W . X^T on v_mfma_f32_32x32x16, a lane owns a token), same LDS
// layout and the same epilogue; the tile is 128 or 256 tokens x one head (a wave owns one or
// two 32-token blocks x the head's four column blocks).  Tiles this small move up to twice
// the LDS bytes per MFMA, and 128-bit LDS stores are slow (13 cycles an instruction against
// 4.7 for a read): here the operand tiles go from memory straight into LDS (buffer loads
// with the LDS bit) through four (three) stages, and the LDS instruction pipe carries the
// operand reads only.
#include "project_epilogue.hpp"

namespace ellm {
namespace proj {
namespace {

constexpr int kMidKc = 64;                        // K elements per chunk: one 128-byte line per row
constexpr int kMidRowPitch = kMidKc * 2;          // unpadded; pieces permuted as in project.hip
// MB = 32-token blocks per wave, WAVES = 4 or 8 waves: the tile is 32 MB WAVES tokens x one head.
// Forms in use: 4 waves x 1 block (128 tokens) and 8 waves x 1 block (256 tokens, two waves per SIMD
// with 180 registers each).  4 waves x 2 blocks (256 tokens, one wave per SIMD with 330 registers: the
// same MFMAs per chunk, 40 % fewer operand reads, but nothing to issue from while the wave waits for
// its operands or at the chunk's barrier) still compiles and measured 7 % slower.
template <int MB, int WAVES>
struct MidShape {
  static_assert((WAVES == 4 && (MB == 1 || MB == 2)) || (WAVES == 8 && MB == 1), "forms of the tile");
  static constexpr int kThreads = 64 * WAVES;
  static constexpr int kTokens = 32 * MB * WAVES;
  static constexpr int kStageBytes = (kTokens + kHeadDim) * kMidRowPitch;  // X rows then W rows: 32 or 48 KB
  static constexpr int kStages = kTokens == 128 ? 4 : 3;   // chunk c in stage c % kStages
  static constexpr int kLdsBytes = kStages * kStageBytes;
  static constexpr int kRowsPerLoad = 8 * WAVES;    // rows one load of every wave moves (1 KB = 8 rows a wave)
  static constexpr int kXLoads = kTokens / kRowsPerLoad, kWLoads = kHeadDim / kRowsPerLoad;
  static constexpr int kLoads = kXLoads + kWLoads;  // 1 KB wave loads per chunk and wave
  static constexpr int kAhead = kStages - 1;        // chunks requested ahead of the one being multiplied
  // loads a wave still has outstanding when its pieces of the next chunk must have landed: the
  // chunks requested after that one (the literal in the kernel's s_waitcnt)
  static constexpr int kMayBePending = (kAhead - 1) * kLoads;
  static_assert(kMayBePending == (WAVES == 8 ? 6 : (MB == 1 ? 16 : 12)), "s_waitcnt vmcnt literals in project_mid_kernel");
  static_assert(WAVES * kEpWaveBytes <= kLdsBytes, "the epilogue reuses the stages");
  static_assert(kLdsBytes <= 160 * 1024, "LDS of a compute unit");
};

template <typename S, int MODE, int MB, int WAVES>
__global__ __launch_bounds__(64 * WAVES) void project_mid_kernel(ProjectKernelArgs p) {
  using M = Mfma<S>;
  using Shape = MidShape<MB, WAVES>;
  constexpr int kStageBytes = Shape::kStageBytes, kStages = Shape::kStages, kLoads = Shape::kLoads;
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
  const uint32_t row0 = tm * Shape::kTokens;
  const uint32_t rows_here = min(p.rows - row0, (uint32_t)Shape::kTokens);
  // (descriptors as four plain words: base, base >> 32, bytes, flags; they go into inline asm)
  auto make_rsrc = [](uint64_t base, uint32_t bytes) {
    return u32x4{(uint32_t)base, (uint32_t)(base >> 32) & 0xffffu, bytes, (uint32_t)kBufFlags};
  };
  const u32x4 x_rsrc = make_rsrc(uniform64(p.x) + (uint64_t)row0 * K * 2, rows_here * K * 2);
  const uint16_t* wbase = p.w[0];
  uint32_t hs = tn;
  if (tn >= p.heads0 + p.heads_kv) {
    wbase = p.w[2];
    hs = tn - p.heads0 - p.heads_kv;
  } else if (tn >= p.heads0) {
    wbase = p.w[1];
    hs = tn - p.heads0;
  }
  const u32x4 w_rsrc = make_rsrc(uniform64(wbase) + (uint64_t)hs * kHeadDim * K * 2, kHeadDim * K * 2);

  // staging: lane l of a wave instruction delivers its 16 bytes to M0 + 16 l, so a wave fills
  // 1 KB = eight whole rows of a stage per instruction; thread -> row tid / 8 (+ 8 WAVES i: the
  // X rows for i < kXLoads, then the 128 W rows), LDS piece tid % 8.  The permutation of the pieces
  // within a row (piece p of row r sits at p ^ ((r >> 1) & 7)) is applied on the memory side:
  // which piece of the line a lane asks for.  Eight lanes still fetch one whole 128-byte line.
  // Rows past the end of the activations read zeros.
  const uint32_t st_row = tid >> 3, st_piece = (tid & 7) ^ ((tid >> 4) & 7);
  constexpr int kXLoads = Shape::kXLoads;
  uint32_t src_off[kXLoads];
#pragma unroll
  for (int i = 0; i < kXLoads; ++i) src_off[i] = (st_row + Shape::kRowsPerLoad * i) * K * 2 + st_piece * 16;
  const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)mid_smem;
  const uint32_t st_wave = lds0 + (uint32_t)__builtin_amdgcn_readfirstlane(wave) * 1024;
  // Written as asm: the compiler's own form of this load makes it wait for every outstanding
  // one before each later LDS read (it cannot see that the two touch different stages).  M0
  // carries the LDS address of the wave's 1 KB; one wait state between its write and the load.
  // (M0 is a register the compiler reserves and, in this kernel, never uses itself.)
  auto load_lds = [](const u32x4& rsrc, uint32_t voff, uint32_t soff, uint32_t lds_at) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                 :: "s"(lds_at), "v"(voff), "s"(rsrc), "s"(soff) : "memory");
  };
  // A chunk past the last one is requested through descriptors of size zero: no memory
  // access, zeros into a stage nobody reads, and every iteration issues the same eight loads.
  const u32x4 none_rsrc = make_rsrc(uniform64(p.x), 0);
  auto load_piece = [&](uint32_t chunk, int i) {
    const uint32_t to = st_wave + (chunk % kStages) * kStageBytes + 1024 * WAVES * i;
    const bool real = chunk < n_chunks;
    load_lds(real ? (i < kXLoads ? x_rsrc : w_rsrc) : none_rsrc, src_off[i < kXLoads ? i : i - kXLoads],
             chunk * (kMidKc * 2), to);
  };

  f32x16 acc[4][MB];  // [column block nb][token block mb]
#pragma unroll
  for (int nb = 0; nb < 4; ++nb)
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[nb][mb][r] = 0.0f;

  // operand reads: lane (j, g) takes row j of a 32-row block, piece 2 step + g, permuted
  const uint32_t swz = (j >> 1) & 7;
  const uint32_t x_row = lds0 + (wave * 32 * MB + j) * kMidRowPitch;
  const uint32_t w_row = lds0 + (Shape::kTokens + j) * kMidRowPitch;
  // operands of one 16-wide step: the wave's MB X blocks (o < MB), then the head's four W blocks
  constexpr int kOps = MB + 4;
  u32x4 ops[2][kOps];
  auto read_operand = [&](auto set_, uint32_t stage, int st, int o) {
    constexpr int set = decltype(set_)::value;
    const uint32_t piece = ((2 * st + g) ^ swz) * 16;
    if (o < MB)
      ops[set][o] = *(const LdsVec4*)(x_row + stage + 32 * o * kMidRowPitch + piece);
    else
      ops[set][o] = *(const LdsVec4*)(w_row + stage + 32 * (o - MB) * kMidRowPitch + piece);
  };

  // prologue: the first kAhead chunks on their way; chunk 0 has landed in every wave's rows
#pragma unroll
  for (int k = 0; k < Shape::kAhead; ++k)
#pragma unroll
    for (int i = 0; i < kLoads; ++i) load_piece(k, i);
  // (requested behind the first chunks, used after the loop: destinations, positions and the
  // first rows of the rotary table or the residual)
  const HeadRows<MB> head = prepare_head<S, MODE, MB>(p, tn, row0 + 32 * MB * wave, lane);
  if constexpr (WAVES == 8)
    asm volatile("s_waitcnt vmcnt(6)" ::: "memory");    // Shape::kMayBePending
  else if constexpr (MB == 1)
    asm volatile("s_waitcnt vmcnt(16)" ::: "memory");
  else
    asm volatile("s_waitcnt vmcnt(12)" ::: "memory");
  __syncthreads();
#pragma unroll
  for (int o = 0; o < kOps; ++o) read_operand(std::integral_constant<int, 0>{}, 0, 0, o);

  // One iteration = one chunk = four 16-wide steps of 4 MB MFMAs.  The operands of a step
  // are read during the step before it, across chunks too.  During steps 0-1 chunk c + kAhead
  // is requested into the stage chunk c - 1 has left; after step 2 the wave waits for its own
  // pieces of chunk c + 1 (all but the loads of the chunks after it) and meets the others at
  // the one barrier of the iteration.  The barrier orders both hazards: the stage being
  // refilled was last read for step 3 of chunk c - 1, and those reads had returned before the
  // previous barrier; and chunk c + 1 is complete before the reads of its first step, issued
  // during step 3.
  constexpr int kPerStep = 4 * MB;
  for (uint32_t c = 0; c < n_chunks; ++c) {
    const uint32_t cur = (c % kStages) * kStageBytes;
    const uint32_t nxt = ((c + 1) % kStages) * kStageBytes;
    __builtin_amdgcn_sched_barrier(0);
    static_for<4 * kPerStep>([&](auto n_) {
      constexpr int n = decltype(n_)::value;
      constexpr int st = n / kPerStep, m = n % kPerStep;
      constexpr int mb = m % MB, nb = m / MB;
      constexpr int set = st & 1;
      acc[nb][mb] = M::m32x32x16(ops[set][MB + nb], ops[set][mb], acc[nb][mb]);
      // the next step's MB + 4 operands, read over this step's MFMAs (two after the first)
      const uint32_t from = (st < 3) ? cur : nxt;
      constexpr int next_st = (st + 1) & 3;
      if constexpr (m == 0) {
        read_operand(std::integral_constant<int, 1 - set>{}, from, next_st, 0);
        read_operand(std::integral_constant<int, 1 - set>{}, from, next_st, MB);
      } else if constexpr (m < kOps - 1) {
        // remaining X blocks first (MB == 2: block 1), then W blocks 1..3
        constexpr int o = (m < MB) ? m : m + 1;
        read_operand(std::integral_constant<int, 1 - set>{}, from, next_st, o);
      }
      if constexpr (n < kLoads) load_piece(c + Shape::kAhead, n);
      if constexpr (n == 3 * kPerStep - 1) {
        // this wave's pieces of chunk c + 1 are in LDS, and its reads of this chunk's stage
        // have returned
        if constexpr (WAVES == 8)
          asm volatile("s_waitcnt vmcnt(6) lgkmcnt(0)" ::: "memory");
        else if constexpr (MB == 1)
          asm volatile("s_waitcnt vmcnt(16) lgkmcnt(0)" ::: "memory");
        else
          asm volatile("s_waitcnt vmcnt(12) lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();
      }
      __builtin_amdgcn_sched_barrier(0);
    });
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the last (empty) requests still write LDS
  __syncthreads();
  finish_head<S, MODE, MB>(p, acc, head, lds0 + wave * kEpWaveBytes, lane);
}

template <int MB, int WAVES>
hipError_t prepare_shape() {
  const void* kernels[] = {(const void*)project_mid_kernel<F16, kModeQkv, MB, WAVES>,
                           (const void*)project_mid_kernel<BF16, kModeQkv, MB, WAVES>,
                           (const void*)project_mid_kernel<F16, kModeAdd, MB, WAVES>,
                           (const void*)project_mid_kernel<BF16, kModeAdd, MB, WAVES>};
  for (const void* k : kernels) {
    const hipError_t e =
        hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, MidShape<MB, WAVES>::kLdsBytes);
    if (e != hipSuccess) return e;
  }
  return hipSuccess;
}

template <int MB, int WAVES>
hipError_t launch_shape(ProjectKernelArgs p, int dtype, bool add, hipStream_t stream) {
  using Shape = MidShape<MB, WAVES>;
  p.tiles_m = (p.rows + Shape::kTokens - 1) / Shape::kTokens;
  p.tiles_n = p.heads0 + 2 * p.heads_kv;
  const uint32_t blocks = p.tiles_m * p.tiles_n;
  auto go = [&](auto kernel) {
    hipLaunchKernelGGL(kernel, dim3(blocks), dim3(Shape::kThreads), Shape::kLdsBytes, stream, p);
    return hipGetLastError();
  };
  if (add)
    return dtype == 0 ? go(project_mid_kernel<F16, kModeAdd, MB, WAVES>) : go(project_mid_kernel<BF16, kModeAdd, MB, WAVES>);
  return dtype == 0 ? go(project_mid_kernel<F16, kModeQkv, MB, WAVES>) : go(project_mid_kernel<BF16, kModeQkv, MB, WAVES>);
}

}  // namespace

hipError_t mid_prepare() {
  const hipError_t e = prepare_shape<1, 4>();
  return e != hipSuccess ? e : prepare_shape<1, 8>();
}

// The 256-token tile runs as eight waves of one token block each: measured against four waves of two
// blocks at 1536 rows x 2048 -> 5120, 36.9 against 39.5 us (either way a compute unit takes in
// (256 + 128) x 128 bytes of operands per chunk at the 55-60 GB/s one unit streams from L2, which is
// what sets the chunk time of 0.8 us; the second wave per SIMD only hides the stalls around it).
hipError_t launch_project_mid(ProjectKernelArgs p, uint32_t token_blocks, int dtype, bool add,
                              hipStream_t stream) {
  if (token_blocks != 2) return launch_shape<1, 4>(p, dtype, add, stream);
  return launch_shape<1, 8>(p, dtype, add, stream);
}

}  // namespace proj
}  // namespace ellm
