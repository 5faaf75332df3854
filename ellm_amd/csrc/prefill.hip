// Causal GQA attention for a chunk of new tokens (position_interval > 1) on
// gfx950 MFMA, FlashAttention-style: K/V tiles staged in LDS, binary32 online
// soft-max in registers, causal tile skipping.
//
// Replaces the (token, sequence, query head) task loop of Attention::run
// (reference: src/compiler/mul/attention.rs:83-153) and its leaf
// flash_attention (src/kernel/x86_64/f16_512/flash_attention.rs:30-92), which
// walks keys 0..=position once per query row.  Same result per row:
// softmax(scale * q.K[0..=position]^T) . V[0..=position].
//
// Formulation (everything transposed so that one lane owns one query row):
//   S^T[key][row] = K . Q^T     32x32x16 MFMA, A = K tile from LDS, B = Q in registers
//   O^T[d][row]  += V^T . P^T   32x32x16 MFMA, A = V^T tile from LDS, B = P^T in registers
// The C layout of S^T (lane = row, registers = keys) is, up to a fixed
// permutation of keys inside each 16-key group, the B layout the second MFMA
// wants; V^T is written to LDS with the same permutation, so P never leaves the
// lane that produced it and row max / row sum need one cross-lane exchange.
//
// A workgroup (4 waves) owns 4*NB blocks of 32 query rows that all read the
// same K/V plane: up to 8 query heads of one GQA group x consecutive token
// blocks.  Stacking the group's heads makes each LDS tile feed 4*NB times more
// MFMA work and keeps the token span (and so the masked part of the diagonal
// tile) short.
#include <cstdlib>

#include "common.hpp"
#include "kernels.hpp"

namespace ellm {
namespace {

constexpr int kPfWaves = 4;
constexpr int kPfThreads = kPfWaves * kWave;
constexpr int kBK = 64;                     // keys per tile
constexpr int kKsPitch = kHeadDim + 8;      // halves per K row (272 B)
constexpr int kVtsPitch = kBK + 8;          // halves per V^T row (144 B)
constexpr int kKsHalves = kBK * kKsPitch;
constexpr int kVtsHalves = kHeadDim * kVtsPitch;
constexpr int kStageHalves = kKsHalves + kVtsHalves;
constexpr float kRescaleStep = 8.0f;        // log2 units

struct PrefillKernelArgs {
  const uint16_t* q;
  const uint16_t* k;
  const uint16_t* v;
  uint16_t* out;
  float* lse;
  size_t q_token_stride;  // elements between consecutive tokens of Q/O
  size_t kv_stride_seq, kv_stride_head, kv_stride_pos;
  uint32_t batch_pitch;
  uint32_t n_q_heads, n_kv_heads, group;
  uint32_t heads_per_wg;     // query heads stacked in one workgroup
  uint32_t tblocks_per_wg;   // 32-token blocks per workgroup
  uint32_t head_groups;      // group / heads_per_wg
  uint32_t n_wg_tokens;      // workgroups along the token axis
  uint32_t combos;           // batch * kv_heads * head_groups
  uint32_t xcd_mode;         // 1: workgroup id % 8 selects the K/V plane
  uint32_t position_index, interval;
  uint32_t negate_q;         // scale < 0: fold the sign into Q (exact) so that c > 0
  float c;                   // |scale| * log2(e), > 0
};

template <typename T, int NB>
__global__ __launch_bounds__(kPfThreads, NB == 1 ? 2 : 1) void prefill_kernel(PrefillKernelArgs p) {
  __shared__ __attribute__((aligned(16))) uint16_t smem[2 * kStageHalves];

  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int j = lane & 31, g = lane >> 5;

  // ---- which (plane, token block) this workgroup owns ----------------------
  // Workgroups are dealt to the 8 XCDs round-robin by id.  When the planes
  // divide 8, id % 8 picks the plane, so each XCD's L2 only ever holds one K/V
  // plane; in every case long rows (late tokens) come first so the tail of the
  // launch is made of short work items.
  uint32_t combo, order;
  if (p.xcd_mode) {
    const uint32_t xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    const uint32_t per = 8 / p.combos;
    combo = xcd % p.combos;
    order = slot * per + xcd / p.combos;
  } else {
    combo = blockIdx.x % p.combos;
    order = blockIdx.x / p.combos;
  }
  if (order >= p.n_wg_tokens) return;
  const uint32_t wg_tok = p.n_wg_tokens - 1 - order;
  const uint32_t seq = combo / (p.n_kv_heads * p.head_groups);
  const uint32_t kvh = (combo / p.head_groups) % p.n_kv_heads;
  const uint32_t hgrp = combo % p.head_groups;
  const uint32_t t_base = wg_tok * 32 * p.tblocks_per_wg;
  const uint32_t S = p.interval, P0 = p.position_index;

  const uint32_t wg_last_tok = min(S, t_base + 32 * p.tblocks_per_wg) - 1;
  const uint32_t kmax = P0 + wg_last_tok;  // last key any row here may see
  const uint32_t n_tiles = kmax / kBK + 1;

  // ---- per row-block bookkeeping -------------------------------------------
  uint32_t head[NB], tok[NB], first_pos[NB], last_pos[NB];
  bool active[NB], row_valid[NB];
#pragma unroll
  for (int n = 0; n < NB; ++n) {
    const uint32_t rb = wave * NB + n;
    const uint32_t hg = rb % p.heads_per_wg, tb = rb / p.heads_per_wg;
    head[n] = kvh * p.group + hgrp * p.heads_per_wg + hg;
    const uint32_t tok0 = t_base + 32 * tb;
    active[n] = tok0 < S;
    tok[n] = min(tok0 + j, S - 1);  // clamped rows compute a valid row and are not stored
    row_valid[n] = tok0 + j < S;
    first_pos[n] = P0 + min(tok0, S - 1);
    last_pos[n] = P0 + min(tok0 + 31, S - 1);
  }

  // ---- Q as the B operand: lane (row j, half g) holds q[row][16 s + 8 g + 0..7] -------
  u32x4 qreg[NB][8];
#pragma unroll
  for (int n = 0; n < NB; ++n) {
    const uint16_t* qrow =
        p.q + (size_t)tok[n] * p.q_token_stride + ((size_t)seq * p.n_q_heads + head[n]) * kHeadDim;
#pragma unroll
    for (int s = 0; s < 8; ++s) {
      qreg[n][s] = load16(qrow + 16 * s + 8 * g);
      if (p.negate_q) qreg[n][s] ^= 0x80008000u;
    }
  }
  const float c = p.c;

  const uint16_t* kplane = p.k + seq * p.kv_stride_seq + kvh * p.kv_stride_head;
  const uint16_t* vplane = p.v + seq * p.kv_stride_seq + kvh * p.kv_stride_head;

  // ---- tile staging: HBM -> registers -> LDS -------------------------------
  const int ld_c = tid & 15;    // 8-element column chunk
  const int ld_r = tid >> 4;    // 0..15
  // V^T column position of the 4-key group this thread transposes: the two low
  // bits of the group index are swapped (see the layout note above).
  const int vt_grp = (ld_r & ~3) | ((ld_r & 1) << 1) | ((ld_r >> 1) & 1);
  // 16-byte chunks of a V^T row are XOR-swizzled with bits 4..6 of the row (d)
  // index: the transposing 8-byte writes (rows 8 apart across lanes) and the
  // 16-byte operand reads (consecutive rows across lanes) are then both free
  // of LDS bank conflicts.
  const int vt_swz = (ld_c >> 1) & 7;
  u32x4 kreg[4], vreg[4];
  auto issue_loads = [&](uint32_t kt) {
    const uint32_t kb = kt * kBK;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t krow = min(kb + ld_r + 16 * i, kmax);
      kreg[i] = load16(kplane + (size_t)krow * p.kv_stride_pos + 8 * ld_c);
      const uint32_t vrow = min(kb + 4 * ld_r + i, kmax);
      vreg[i] = load16(vplane + (size_t)vrow * p.kv_stride_pos + 8 * ld_c);
    }
  };
  auto store_tile = [&](int buf) {
    uint16_t* ks = smem + buf * kStageHalves;
    uint16_t* vts = ks + kKsHalves;
#pragma unroll
    for (int i = 0; i < 4; ++i) store16(ks + (ld_r + 16 * i) * kKsPitch + 8 * ld_c, kreg[i]);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      u32x2 col = gather_column(vreg[0][e >> 1], vreg[1][e >> 1], vreg[2][e >> 1],
                                vreg[3][e >> 1], (e & 1) != 0);
      *(u32x2*)(vts + (8 * ld_c + e) * kVtsPitch + 8 * ((vt_grp >> 1) ^ vt_swz) +
                4 * (vt_grp & 1)) = col;
    }
  };

  float m_run[NB], l_run[NB];
  f32x16 oacc[NB][4];
#pragma unroll
  for (int n = 0; n < NB; ++n) {
    m_run[n] = -INFINITY;
    l_run[n] = 0.0f;
#pragma unroll
    for (int db = 0; db < 4; ++db)
#pragma unroll
      for (int r = 0; r < 16; ++r) oacc[n][db][r] = 0.0f;
  }

  issue_loads(0);
  store_tile(0);
  __syncthreads();

  for (uint32_t kt = 0; kt < n_tiles; ++kt) {
    const int buf = kt & 1;
    const bool more = kt + 1 < n_tiles;
    if (more) issue_loads(kt + 1);

    const uint16_t* ks = smem + buf * kStageHalves;
    const uint16_t* vts = ks + kKsHalves;
    const uint32_t kb = kt * kBK;

    bool any_active = false;
#pragma unroll
    for (int n = 0; n < NB; ++n) any_active |= active[n] && kb <= last_pos[n];

    if (any_active) {
      // ---- S^T = K . Q^T ----------------------------------------------------
      f32x16 st[NB][2];
#pragma unroll
      for (int n = 0; n < NB; ++n)
#pragma unroll
        for (int mb = 0; mb < 2; ++mb)
#pragma unroll
          for (int r = 0; r < 16; ++r) st[n][mb][r] = 0.0f;
#pragma unroll
      for (int s = 0; s < 8; ++s) {
#pragma unroll
        for (int mb = 0; mb < 2; ++mb) {
          const u32x4 a = load16(ks + (32 * mb + j) * kKsPitch + 16 * s + 8 * g);
#pragma unroll
          for (int n = 0; n < NB; ++n) st[n][mb] = Mfma<T>::m32x32x16(a, qreg[n][s], st[n][mb]);
        }
      }

      // ---- online soft-max, one query row per lane --------------------------
      // Scores stay unscaled; scale*log2(e) (c > 0) is folded into the exponent's
      // FMA.  The reference max m is only moved when the tile's max exceeds it by
      // more than kRescaleStep (log2 units), so most tiles skip the rescale of
      // O^T; probabilities are then at most 2^kRescaleStep, well inside binary16
      // and bfloat16 range.  The row sum adds the unrounded binary32
      // probabilities: summing the rounded ones is cheaper but moves the
      // log-sum-exp by up to half a storage ulp, beyond its 1e-4 tolerance.
      u32x4 pk[NB][4];
#pragma unroll
      for (int n = 0; n < NB; ++n) {
        if (kb + kBK - 1 > first_pos[n]) {  // tile crosses this block's diagonal
          const uint32_t rowpos = P0 + tok[n];
#pragma unroll
          for (int mb = 0; mb < 2; ++mb)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
              const uint32_t key = kb + 32 * mb + 8 * (r >> 2) + 4 * g + (r & 3);
              st[n][mb][r] = (key <= rowpos) ? st[n][mb][r] : -INFINITY;
            }
        }
        float rmax = st[n][0][0];
#pragma unroll
        for (int mb = 0; mb < 2; ++mb)
#pragma unroll
          for (int r = 0; r < 16; ++r) rmax = fmaxf(rmax, st[n][mb][r]);
        rmax = fmaxf(rmax, xor_shuffle(rmax, 32));
        const float tmax = rmax * c;
        const bool grow = tmax > m_run[n] + kRescaleStep;
        if (__any(grow)) {
          const float m_new = grow ? tmax : m_run[n];
          const float alpha = grow ? fast_exp2(m_run[n] - m_new) : 1.0f;
          m_run[n] = m_new;
          l_run[n] *= alpha;
#pragma unroll
          for (int db = 0; db < 4; ++db) oacc[n][db] *= alpha;
        }
        // m_run is finite from tile 0 on (key 0 is visible to every row); the
        // guard only keeps -inf - -inf out of the arithmetic.
        const float neg_m = (m_run[n] == -INFINITY) ? 0.0f : -m_run[n];
        float psum = 0.0f;
#pragma unroll
        for (int cc = 0; cc < 4; ++cc) {
          const int mb = cc >> 1, r0 = 8 * (cc & 1);
#pragma unroll
          for (int w = 0; w < 4; ++w) {
            const float p0 = fast_exp2(__builtin_fmaf(st[n][mb][r0 + 2 * w], c, neg_m));
            const float p1 = fast_exp2(__builtin_fmaf(st[n][mb][r0 + 2 * w + 1], c, neg_m));
            const uint32_t word = Mfma<T>::pack2(p0, p1);
            pk[n][cc][w] = word;
            psum += p0 + p1;
          }
        }
        l_run[n] += psum;
      }

      // ---- O^T += V^T . P^T --------------------------------------------------
#pragma unroll
      for (int cc = 0; cc < 4; ++cc) {
#pragma unroll
        for (int db = 0; db < 4; ++db) {
          const int chunk = (2 * cc + g) ^ ((2 * db + (j >> 4)) & 7);
          const u32x4 a = load16(vts + (32 * db + j) * kVtsPitch + 8 * chunk);
#pragma unroll
          for (int n = 0; n < NB; ++n) oacc[n][db] = Mfma<T>::m32x32x16(a, pk[n][cc], oacc[n][db]);
        }
      }
    }

    if (more) store_tile(buf ^ 1);
    __syncthreads();
  }

  // ---- epilogue: normalise, convert, store ----------------------------------
#pragma unroll
  for (int n = 0; n < NB; ++n) {
    float l = l_run[n] + xor_shuffle(l_run[n], 32);
    if (!(active[n] && row_valid[n])) continue;
    const float inv = 1.0f / l;
    uint16_t* orow =
        p.out + (size_t)tok[n] * p.q_token_stride + ((size_t)seq * p.n_q_heads + head[n]) * kHeadDim;
#pragma unroll
    for (int db = 0; db < 4; ++db)
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {
        u32x2 w;
        w[0] = Mfma<T>::pack2(oacc[n][db][4 * q4] * inv, oacc[n][db][4 * q4 + 1] * inv);
        w[1] = Mfma<T>::pack2(oacc[n][db][4 * q4 + 2] * inv, oacc[n][db][4 * q4 + 3] * inv);
        *(u32x2*)(orow + 32 * db + 8 * q4 + 4 * g) = w;
      }
    if (p.lse && g == 0)
      p.lse[((size_t)tok[n] * p.batch_pitch + seq) * p.n_q_heads + head[n]] =
          (m_run[n] + fast_log2(l)) * kLn2;
  }
}

uint32_t gcd_u32(uint32_t a, uint32_t b) {
  while (b) {
    const uint32_t t = a % b;
    a = b;
    b = t;
  }
  return a;
}

template <typename T, int NB>
hipError_t launch_nb(const AttnArgs& a, hipStream_t stream) {
  constexpr uint32_t kRowBlocks = kPfWaves * NB;
  PrefillKernelArgs p;
  p.q = (const uint16_t*)a.q;
  p.k = (const uint16_t*)a.k;
  p.v = (const uint16_t*)a.v;
  p.out = (uint16_t*)a.out;
  p.lse = a.lse;
  p.q_token_stride = (size_t)a.batch_pitch * a.n_q_heads * kHeadDim;
  p.kv_stride_seq = a.kv_stride_seq;
  p.kv_stride_head = a.kv_stride_head;
  p.kv_stride_pos = a.kv_stride_pos;
  p.batch_pitch = a.batch_pitch;
  p.n_q_heads = a.n_q_heads;
  p.n_kv_heads = a.n_kv_heads;
  p.group = a.group;
  p.heads_per_wg = gcd_u32(a.group, kRowBlocks);
  p.tblocks_per_wg = kRowBlocks / p.heads_per_wg;
  p.head_groups = a.group / p.heads_per_wg;
  const uint32_t wg_tokens = 32 * p.tblocks_per_wg;
  p.n_wg_tokens = (a.position_interval + wg_tokens - 1) / wg_tokens;
  p.combos = a.batch * a.n_kv_heads * p.head_groups;
  p.xcd_mode = (p.combos <= 8 && 8 % p.combos == 0) ? 1 : 0;
  p.position_index = a.position_index;
  p.interval = a.position_interval;
  float c = a.scale * kLog2e;
  p.negate_q = c < 0.0f ? 1u : 0u;
  c = c < 0.0f ? -c : c;
  // scale == 0 (uniform attention): a tiny positive c keeps -inf * c == -inf for masked keys
  p.c = c > 0.0f ? c : 1e-37f;

  uint32_t n_wg;
  if (p.xcd_mode) {
    const uint32_t per = 8 / p.combos;
    n_wg = 8 * ((p.n_wg_tokens + per - 1) / per);
  } else {
    n_wg = p.combos * p.n_wg_tokens;
  }
  hipLaunchKernelGGL((prefill_kernel<T, NB>), dim3(n_wg), dim3(kPfThreads), 0, stream, p);
  return hipGetLastError();
}

}  // namespace

hipError_t launch_prefill(const AttnArgs& a, hipStream_t stream) {
  static const int nb = [] {
    const char* e = getenv("ELLM_PREFILL_NB");
    return (e && e[0] == '1') ? 1 : 2;
  }();
  if (nb == 1) {
    if (a.dtype == 0) return launch_nb<F16, 1>(a, stream);
    return launch_nb<BF16, 1>(a, stream);
  }
  if (a.dtype == 0) return launch_nb<F16, 2>(a, stream);
  return launch_nb<BF16, 2>(a, stream);
}

}  // namespace ellm
