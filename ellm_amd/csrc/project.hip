// Projections around the attention operator on gfx950 MFMA:
//   fused Q/K/V projection   C = X . [Wq; Wk; Wv]^T  with, per finished 128-wide head
//   row, RMS norm (weight 1) and rotary rotation for the query and key heads, the
//   query rows written to the Q scratch, key and value rows written straight to their
//   token coordinates of the cache; replaces MatMul3::run (reference:
//   src/compiler/mul/matmul3.rs:289-385, finalize :243-254 and :436-451);
//   output projection + residual   Y = A . Wo^T + R; replaces MatMulAdd::run
//   (src/compiler/mul/matmul_add.rs:128-232).
// Weights are row-major [N][K] as the reference keeps them ("W_nt"), activations are
// row-major [rows][K]; both operands are K-contiguous, which is what MFMA wants.
//
// Formulation: the product is computed transposed, C^T[n][token] = W . X^T, so that a
// lane of the 32x32 accumulator block owns one token and 16 of 32 output columns: a
// head row (128 columns) of a token then sits in two lanes (l and l ^ 32), the sum of
// squares needs one cross-lane exchange and the (even, odd) rotation pairs are
// register neighbours.
//
// A workgroup of 4 waves (one per SIMD, 512 registers each) owns a tile of 256 tokens x
// 256 output columns (two heads); wave (wn, wm) owns head wn and tokens 128 wm..+127 as
// 4 x 4 accumulator blocks (256 accumulator registers).  K runs in chunks of 64 (one
// 128-byte cache line per operand row and chunk: a fetch of half a line costs the vector
// cache the same miss entry as a whole one) through two LDS stages: chunk c is read while
// chunk c + 1, fetched into registers an iteration earlier, is written to the other stage.
// Calls with at most 64 rows go to the streaming kernel of project_small.hip, calls that would
// leave these tiles fewer than the compute units to the 128-token tiles of project_mid.hip.
#include "project_epilogue.hpp"

namespace ellm {
using namespace proj;
namespace {

constexpr int kTile = 256;                          // tokens, and output columns, per workgroup
constexpr int kKc = 64;                             // K elements per chunk: one 128-byte line per row
// A row of a stage is the chunk's 128 bytes, unpadded; its eight 16-byte pieces are stored
// permuted, piece p of row r at p ^ ((r >> 1) & 7): the 16 lanes of a staging store (two
// whole rows) and the 16 lanes of an operand read (one piece of 16 consecutive rows) then
// both touch every LDS bank once.
constexpr int kRowPitch = kKc * 2;
constexpr int kStageBytes = 2 * kTile * kRowPitch;  // X rows then W rows
constexpr int kStages = 2;
constexpr int kProjThreads = 256;
constexpr int kProjLdsBytes = kStages * kStageBytes;
static_assert(4 * kEpWaveBytes <= kProjLdsBytes, "the epilogue reuses the stages");
constexpr int kGroupM = 4;                          // token tiles that take turns on one column tile


template <typename S, int MODE>
__global__ __launch_bounds__(kProjThreads) void project_kernel(ProjectKernelArgs p) {
  using M = Mfma<S>;
  extern __shared__ __attribute__((aligned(16))) uint8_t proj_smem[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int j = lane & 31, g = lane >> 5;
  const int wn = wave & 1, wm = wave >> 1;

  // workgroup -> tile: ids that share id % 8 (one XCD, one L2) are made consecutive,
  // then kGroupM token tiles x all column tiles form a band that is walked token-first
  uint32_t tm, tn;
  {
    const uint32_t total = p.tiles_m * p.tiles_n;
    const uint32_t q = total >> 3, r = total & 7, xcd = blockIdx.x & 7, idx = blockIdx.x >> 3;
    const uint32_t pid = xcd * q + min(xcd, r) + idx;
    const uint32_t per_band = kGroupM * p.tiles_n;
    const uint32_t band = pid / per_band, in_band = pid % per_band;
    const uint32_t first_m = band * kGroupM;
    const uint32_t band_m = min(p.tiles_m - first_m, (uint32_t)kGroupM);
    tm = first_m + in_band % band_m;
    tn = in_band / band_m;
  }
  const uint32_t heads_total = p.heads0 + 2 * p.heads_kv;
  const uint32_t K = p.K;
  const uint32_t n_chunks = K / kKc;

  // operand sources: one descriptor for the token rows, one per head of the tile
  const uint32_t row0 = tm * kTile;
  const uint32_t rows_here = min(p.rows - row0, (uint32_t)kTile);
  const __amdgpu_buffer_rsrc_t x_rsrc = __builtin_amdgcn_make_buffer_rsrc(
      (void*)(uniform64(p.x) + (uint64_t)row0 * K * 2), 0, rows_here * K * 2, kBufFlags);
  auto head_rsrc = [&](uint32_t hh) {
    const uint16_t* base = p.w[0];
    uint32_t hs = hh, bytes = kHeadDim * K * 2;
    if (hh >= p.heads0 + p.heads_kv) {
      base = p.w[2];
      hs = hh - p.heads0 - p.heads_kv;
    } else if (hh >= p.heads0) {
      base = p.w[1];
      hs = hh - p.heads0;
    }
    if (hh >= heads_total) {  // odd head count: the tile's second half reads zeros
      base = p.w[0];
      hs = 0;
      bytes = 0;
    }
    return __builtin_amdgcn_make_buffer_rsrc((void*)(uniform64(base) + (uint64_t)hs * kHeadDim * K * 2),
                                             0, bytes, kBufFlags);
  };
  const __amdgpu_buffer_rsrc_t w_rsrc0 = head_rsrc(2 * tn), w_rsrc1 = head_rsrc(2 * tn + 1);

  // staging: thread -> row tid / 8 (+ 32 i), 16-byte piece tid % 8 of the chunk's 128 B:
  // eight lanes fetch one whole cache line
  const uint32_t st_row = tid >> 3, st_piece = tid & 7;
  uint32_t src_off[8];  // rows st_row + 32 i of a 256-row (X) or, i & 3, 128-row (W head) source
#pragma unroll
  for (int i = 0; i < 8; ++i) src_off[i] = (st_row + 32 * i) * K * 2 + st_piece * 16;
  const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)proj_smem;
  auto pin = [](uint32_t addr) {
    asm volatile("" : "+v"(addr));
    return addr;
  };
  const uint32_t st_store = lds0 + st_row * kRowPitch + ((st_piece ^ ((st_row >> 1) & 7)) * 16);
  // A chunk is requested one iteration (64 MFMAs, about 1.2 us) before it is stored to LDS.
  u32x4 stg[16];
  // (a chunk past the last one fetches bytes of the next row, or zeros past the end of
  // the buffer, into a stage nobody reads)
  auto load_piece = [&](uint32_t chunk, int i) {
    const uint32_t soff = chunk * (kKc * 2);
    if (i < 8)
      stg[i] = __builtin_amdgcn_raw_buffer_load_b128(x_rsrc, src_off[i], soff, 0);
    else
      stg[i] = __builtin_amdgcn_raw_buffer_load_b128((i < 12) ? w_rsrc0 : w_rsrc1, src_off[i & 3], soff, 0);
  };
  auto store_piece = [&](uint32_t base, int i) {
    *(LdsVec4*)(base + 32 * i * kRowPitch) = stg[i];
  };

  f32x16 acc[4][4];  // [column block nb][token block mb]
#pragma unroll
  for (int nb = 0; nb < 4; ++nb)
#pragma unroll
    for (int mb = 0; mb < 4; ++mb)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[nb][mb][r] = 0.0f;

  // operand reads: lane (j, g) takes row j of a 32-row block, piece 2 step + g of the row,
  // permuted with the row's key; the four steps of a chunk have their own lane addresses
  const uint32_t swz = (j >> 1) & 7;
  uint32_t x_read[4], w_read[4];
#pragma unroll
  for (int st = 0; st < 4; ++st) {
    x_read[st] = lds0 + (wm * 128 + j) * kRowPitch + (((2 * st + g) ^ swz) * 16);
    w_read[st] = lds0 + (kTile + wn * 128 + j) * kRowPitch + (((2 * st + g) ^ swz) * 16);
  }
  // operand o of a step: 0 = W block 0, 1..4 = X blocks, 5..7 = W blocks 1..3 (the order
  // in which the step's MFMAs first need them)
  auto read_operand = [&](uint32_t xb, uint32_t wb, int o) {
    const uint32_t at = (o == 0) ? wb : (o < 5 ? xb + 32 * (o - 1) * kRowPitch : wb + 32 * (o - 4) * kRowPitch);
    return (u32x4) * (const LdsVec4*)at;
  };
  // MFMA n of a step: W block n / 4 times X block n % 4
  auto w_of = [](int n) { return (n >> 2) == 0 ? 0 : 4 + (n >> 2); };
  auto x_of = [](int n) { return 1 + (n & 3); };

  // prologue: chunk 0 into stage 0, chunk 1 into the staging registers
#pragma unroll
  for (int i = 0; i < 16; ++i) load_piece(0, i);
  {
    const uint32_t base = pin(st_store);
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      store_piece(base, i);
      load_piece(1, i);
    }
  }
  __syncthreads();

  // One iteration = one chunk: four 16-wide steps, 64 MFMAs.  Chunk c sits in stage c % 2;
  // during its first three steps the staging registers (chunk c + 1) are stored to the other
  // stage and refilled with chunk c + 2; the iteration's one barrier stands before step 3, and
  // the operands of the next chunk's first step are read, from the stage just completed, during
  // step 3.  So the operands of every step are read during the step before it, across chunks
  // too.  The barrier orders both hazards: the stage being refilled was last read for step 3 of
  // chunk c - 1, and those reads had returned before the previous barrier.
  // LDS traffic is spread evenly (a read every second MFMA, a store every third): the four
  // waves together keep the LDS pipe busy most of the time, and a burst of stores
  // would still be draining when the barrier is reached.
  u32x4 opa[8], opb[8];
#pragma unroll
  for (int o = 0; o < 8; ++o) opa[o] = read_operand(x_read[0], w_read[0], o);
  for (uint32_t c = 0; c < n_chunks; ++c) {
    const uint32_t cur = (c & 1) * kStageBytes, nxt = kStageBytes - cur;
    uint32_t xb[5], wb[5];   // [4]: first step of the next chunk
#pragma unroll
    for (int st = 1; st < 4; ++st) {
      xb[st] = pin(x_read[st] + cur);
      wb[st] = pin(w_read[st] + cur);
    }
    xb[4] = pin(x_read[0] + nxt);
    wb[4] = pin(w_read[0] + nxt);
    const uint32_t store_at = pin(st_store + nxt);
    __builtin_amdgcn_sched_barrier(0);
    static_for<64>([&](auto n_) {
      constexpr int n = decltype(n_)::value;
      constexpr int st = n >> 4, m = n & 15;
      if constexpr ((st & 1) == 0) {
        acc[m >> 2][m & 3] = M::m32x32x16(opa[w_of(m)], opa[x_of(m)], acc[m >> 2][m & 3]);
        if constexpr ((n & 1) == 0) opb[m >> 1] = read_operand(xb[st + 1], wb[st + 1], m >> 1);
      } else {
        acc[m >> 2][m & 3] = M::m32x32x16(opb[w_of(m)], opb[x_of(m)], acc[m >> 2][m & 3]);
        if constexpr ((n & 1) == 0) opa[m >> 1] = read_operand(xb[st + 1], wb[st + 1], m >> 1);
      }
      if constexpr (n < 48 && n % 3 == 2) {
        store_piece(store_at, n / 3);
        load_piece(c + 2, n / 3);
      }
      if constexpr (n == 47) {
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        __builtin_amdgcn_s_barrier();
      }
      __builtin_amdgcn_sched_barrier(0);
    });
  }
  __syncthreads();   // every wave is past its last operand reads: the epilogue reuses the stages

  const HeadRows<4> head = prepare_head<S, MODE, 4>(p, 2 * tn + wn, row0 + wm * 128, lane);
  finish_head<S, MODE, 4>(p, acc, head, lds0 + wave * kEpWaveBytes, lane);
}

}  // namespace

// Compute units of the device the kernels were prepared on (project_prepare()).
static uint32_t g_n_cu = 256;

// Which kernel a call runs: the few-rows streaming kernel when the handle has its workspace
// and the shape fits it; else the smallest tile whose workgroups all fit the part at once, one
// per compute unit (128 tokens x one head, then 256 tokens x one head); else 256 x 256 tiles,
// whose traffic per flop is the lowest.  Measured on 256 compute units for 2048 -> 5120: 128-token
// tiles 20 us up to 768 rows, 256-token tiles 38-42 us up to 1536 rows (128-token tiles in two
// rounds: 40-44 us), 256 x 256 tiles 58 us at 2048 rows (61 and 70 us for the other two).
int project_path(uint32_t rows, uint32_t heads, uint32_t K, bool has_workspace) {
  if (has_workspace && small_kernel_takes(rows, K)) return kPathFewRows;
  if (((rows + 127) / 128) * heads <= g_n_cu) return kPathTiles128;
  if (((rows + 255) / 256) * heads <= g_n_cu) return kPathTiles256x1;
  return kPathTiles;
}

bool project_raw_takes(uint32_t rows, uint32_t heads, uint32_t K, bool has_workspace) {
  return project_path(rows, heads, K, has_workspace) == kPathFewRows;
}

hipError_t launch_project(const ProjectArgs& a, hipStream_t stream) {
  if (a.rows == 0) return hipSuccess;
  ProjectKernelArgs p;
  p.x = (const uint16_t*)a.x;
  p.w[0] = (const uint16_t*)a.w0;
  p.w[1] = (const uint16_t*)a.wk;
  p.w[2] = (const uint16_t*)a.wv;
  p.out0 = (uint16_t*)a.out0;
  p.residual = (const uint16_t*)a.residual;
  p.k_out = (uint16_t*)a.k_out;
  p.v_out = (uint16_t*)a.v_out;
  p.rope = (const uint16_t*)a.rope;
  p.positions = a.positions;
  p.seq_offsets = a.seq_offsets;
  p.seq_caps = a.seq_caps;
  p.kv_stride_seq = a.kv_stride_seq;
  p.kv_stride_head = a.kv_stride_head;
  p.kv_stride_pos = a.kv_stride_pos;
  p.ld0 = a.heads0 * kHeadDim;
  p.rope_pos_stride = a.rope_pos_stride;
  p.rope_head_stride = a.rope_head_stride;
  p.K = a.K;
  p.rows = a.rows;
  p.batch_pitch = a.batch_pitch;
  p.batch = a.batch;
  p.heads0 = a.heads0;
  p.heads_kv = a.heads_kv;
  p.tiles_m = (a.rows + kTile - 1) / kTile;
  p.tiles_n = (a.heads0 + 2 * a.heads_kv + 1) / 2;
  p.position_index = a.position_index;
  p.max_start = a.max_start;
  p.finalize0 = a.finalize0;
  p.eps = a.eps;
  const int path = project_path(a.rows, a.heads0 + 2 * a.heads_kv, a.K, a.ws && a.counters);
  if (a.raw_out) {
    if (path != kPathFewRows || a.residual) return hipErrorInvalidValue;   // (project_raw_takes() said otherwise)
    return launch_project_small(p, a.ws, a.counters, a.dtype, kModeRaw, stream);
  }
  if (path == kPathFewRows)
    return launch_project_small(p, a.ws, a.counters, a.dtype, a.residual ? kModeAdd : kModeQkv, stream);
  if (path == kPathTiles128 || path == kPathTiles256x1)
    return launch_project_mid(p, path == kPathTiles128 ? 1 : 2, a.dtype, a.residual != nullptr, stream);
  const uint32_t blocks = p.tiles_m * p.tiles_n;
  auto go = [&](auto kernel) {
    hipLaunchKernelGGL(kernel, dim3(blocks), dim3(kProjThreads), kProjLdsBytes, stream, p);
    return hipGetLastError();
  };
  if (a.residual)
    return a.dtype == 0 ? go(project_kernel<F16, kModeAdd>) : go(project_kernel<BF16, kModeAdd>);
  return a.dtype == 0 ? go(project_kernel<F16, kModeQkv>) : go(project_kernel<BF16, kModeQkv>);
}

// The kernels' LDS needs exceed the default limit; raised here, on the current device, when
// a handle is created, not at launch (a launch may be recorded into a graph).
hipError_t project_prepare() {
  const void* kernels[] = {(const void*)project_kernel<F16, kModeQkv>, (const void*)project_kernel<BF16, kModeQkv>,
                           (const void*)project_kernel<F16, kModeAdd>, (const void*)project_kernel<BF16, kModeAdd>};
  for (const void* k : kernels) {
    const hipError_t e = hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, kProjLdsBytes);
    if (e != hipSuccess) return e;
  }
  int dev = 0, n_cu = 0;
  if (hipGetDevice(&dev) == hipSuccess &&
      hipDeviceGetAttribute(&n_cu, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n_cu > 0)
    g_n_cu = (uint32_t)n_cu;
  const hipError_t e = mid_prepare();
  if (e != hipSuccess) return e;
  return small_prepare();
}

size_t project_workspace_floats(uint32_t heads, uint32_t K) {
  return small_workspace_floats(heads, K);
}

}  // namespace ellm
