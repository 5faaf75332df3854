// Single-token attention over the static K/V cache (position_interval == 1):
// split-KV streaming kernel + log-sum-exp merge.
//
// Replaces, for one new query per sequence, the per-(sequence, query head) calls of
// flash_attention (reference: src/kernel/x86_64/f16_512/flash_attention.rs:30-92)
// scheduled by Attention::run (src/compiler/mul/attention.rs:83-153).  The
// reference re-streams a K/V plane once per query head; here the heads of a GQA
// group share every K/V row, so each plane is read from HBM once.
//
// Work decomposition
//   grid = (split, kv_head * head_groups, sequence); 256 threads = 4 waves.
//   A split owns keys [split*split_len, (split+1)*split_len) of one plane.  The
//   four waves take alternating 16-key chunks; each wave streams its chunks
//   HBM -> registers (128-bit loads, four full 256-byte rows per instruction)
//   -> its private LDS slice -> MFMA operands, so no workgroup barrier is needed
//   inside the loop.  Scores S^T[key][head] = K.Q^T use 16x16x32 MFMA with up to
//   16 query heads in the N dimension; O^T[d][head] += V^T.P^T uses 16x16x16 MFMA,
//   whose B-operand layout is exactly the C layout S^T comes out in.
//   V is transposed on the way into LDS with 4-key x 8-dim register blocks.
//   Soft-max state (running max, denominator) is one scalar per lane.
//   At the end the four waves are merged through LDS; with more than one split
//   the partial (max, sum, acc[128]) goes to the workspace and merge_kernel
//   combines the splits.
#include "common.hpp"
#include "kernels.hpp"

namespace ellm {
namespace {

constexpr int kDecWaves = 4;
constexpr int kChunk = 16;                      // keys per wave step
constexpr int kKPitch = kHeadDim + 8;           // halves per K row in LDS (272 B)
constexpr int kVtPitch = kChunk + 4;            // halves per V^T row in LDS (40 B)
constexpr int kWaveLdsHalves = kChunk * kKPitch + kHeadDim * kVtPitch;
constexpr int kMaxHeadsPerGroup = 16;

struct DecodeKernelArgs {
  const uint16_t* q;
  const uint16_t* k;
  const uint16_t* v;
  uint16_t* out;
  float* lse;
  const uint32_t* positions;
  float* ws_acc;
  float* ws_ml;
  size_t kv_stride_seq, kv_stride_head, kv_stride_pos;
  uint32_t n_q_heads, n_kv_heads, group, head_groups;
  uint32_t position;  // shared position (positions == null) or upper bound
  uint32_t split_len, n_split;
  float scale_log2;   // scale * log2(e)
};

template <typename T>
__global__ __launch_bounds__(kDecWaves* kWave) void decode_split_kernel(DecodeKernelArgs p) {
  __shared__ __attribute__((aligned(16))) uint16_t smem[kDecWaves * kWaveLdsHalves];

  const uint32_t split = blockIdx.x;
  const uint32_t kvh = blockIdx.y / p.head_groups;
  const uint32_t hgrp = blockIdx.y % p.head_groups;
  const uint32_t seq = blockIdx.z;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int g = lane >> 4, c = lane & 15;

  uint32_t pos = p.position;
  if (p.positions) pos = min(p.positions[seq], p.position);
  const uint32_t len = pos + 1;
  const uint32_t k_begin = split * p.split_len;
  const uint32_t k_end = min(len, k_begin + p.split_len);
  const uint32_t heads_here = min((uint32_t)kMaxHeadsPerGroup, p.group - hgrp * kMaxHeadsPerGroup);
  // A split that starts beyond this sequence's keys has nothing to add; the
  // merge kernel derives the number of live splits from the same length.
  if (k_begin >= len) return;

  const uint16_t* kplane = p.k + seq * p.kv_stride_seq + kvh * p.kv_stride_head;
  const uint16_t* vplane = p.v + seq * p.kv_stride_seq + kvh * p.kv_stride_head;

  // Query heads of this group as the B operand of S^T = K.Q^T:
  // lane (head c, group g) holds q[head][32 s + 8 g + 0..7] for s = 0..3.
  const uint32_t head0 = kvh * p.group + hgrp * kMaxHeadsPerGroup;
  u32x4 qreg[4];
  {
    const uint16_t* qrow = p.q + ((size_t)seq * p.n_q_heads + head0 + c) * kHeadDim;
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      if ((uint32_t)c < heads_here)
        qreg[s] = load16(qrow + 32 * s + 8 * g);
      else
        qreg[s] = u32x4{0, 0, 0, 0};
    }
  }

  uint16_t* ks = smem + wave * kWaveLdsHalves;  // [16][kKPitch]
  uint16_t* vt = ks + kChunk * kKPitch;         // [128][kVtPitch]

  const uint32_t n_chunks = (k_end - k_begin + kChunk - 1) / kChunk;
  u32x4 kreg[4], vreg[4];
  auto issue_loads = [&](uint32_t chunk) {
    const uint32_t kb = k_begin + chunk * kChunk;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      // rows past the last valid key are clamped onto it: always in bounds,
      // always initialised, and their probabilities are forced to zero below.
      const uint32_t row = min(kb + 4 * g + i, pos);
      kreg[i] = load16(kplane + (size_t)row * p.kv_stride_pos + 8 * c);
      vreg[i] = load16(vplane + (size_t)row * p.kv_stride_pos + 8 * c);
    }
  };

  float m_run = -INFINITY;  // running max, log2 units (score * scale * log2 e)
  float l_run = 0.0f;       // this lane's share of the denominator
  f32x4 acc[8];
#pragma unroll
  for (int b = 0; b < 8; ++b) acc[b] = f32x4{0, 0, 0, 0};

  uint32_t chunk = wave;
  if (chunk < n_chunks) issue_loads(chunk);
  for (; chunk < n_chunks; chunk += kDecWaves) {
    const uint32_t kb = k_begin + chunk * kChunk;
    // registers -> LDS: K row-major, V transposed.
#pragma unroll
    for (int i = 0; i < 4; ++i) store16(ks + (4 * g + i) * kKPitch + 8 * c, kreg[i]);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      u32x2 col = gather_column(vreg[0][e >> 1], vreg[1][e >> 1], vreg[2][e >> 1],
                                vreg[3][e >> 1], (e & 1) != 0);
      *(u32x2*)(vt + (8 * c + e) * kVtPitch + 4 * g) = col;
    }
    if (chunk + kDecWaves < n_chunks) issue_loads(chunk + kDecWaves);
    __builtin_amdgcn_wave_barrier();

    // S^T[key][head], lane (head c, group g) register r <-> key kb + 4 g + r.
    f32x4 st = {0, 0, 0, 0};
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      u32x4 a = load16(ks + c * kKPitch + 32 * s + 8 * g);
      st = Mfma<T>::m16x16x32(a, qreg[s], st);
    }
    float t[4];
    float tmax = -INFINITY;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      t[r] = (kb + 4 * g + r <= pos) ? st[r] * p.scale_log2 : -INFINITY;
      tmax = fmaxf(tmax, t[r]);
    }
    tmax = fmaxf(tmax, xor_shuffle(tmax, 16));
    tmax = fmaxf(tmax, xor_shuffle(tmax, 32));
    const float m_new = fmaxf(m_run, tmax);  // finite: key kb is always valid
    const float alpha = fast_exp2(m_run - m_new);
    float pr[4];
    float psum = 0.0f;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      pr[r] = fast_exp2(t[r] - m_new);
      psum += pr[r];
    }
    l_run = l_run * alpha + psum;
    m_run = m_new;
    u32x2 pb;
    pb[0] = Mfma<T>::pack2(pr[0], pr[1]);
    pb[1] = Mfma<T>::pack2(pr[2], pr[3]);
#pragma unroll
    for (int b = 0; b < 8; ++b) {
      acc[b] *= alpha;
      u32x2 a = *(const u32x2*)(vt + (16 * b + c) * kVtPitch + 4 * g);
      acc[b] = Mfma<T>::m16x16x16(a, pb, acc[b]);
    }
    __builtin_amdgcn_wave_barrier();
  }

  l_run += xor_shuffle(l_run, 16);
  l_run += xor_shuffle(l_run, 32);

  // Merge the four waves through LDS: red[wave][head][128 acc + max + sum].
  __syncthreads();
  float* red = (float*)smem;
  constexpr int kRedPitch = kHeadDim + 2;
  static_assert(kDecWaves * kMaxHeadsPerGroup * kRedPitch * 4 <= kDecWaves * kWaveLdsHalves * 2,
                "reduction buffer must fit in the staging buffers");
  if ((uint32_t)c < heads_here) {
    float* row = red + (wave * kMaxHeadsPerGroup + c) * kRedPitch;
#pragma unroll
    for (int b = 0; b < 8; ++b)
#pragma unroll
      for (int r = 0; r < 4; ++r) row[16 * b + 4 * g + r] = acc[b][r];
    if (g == 0) {
      row[kHeadDim] = m_run;
      row[kHeadDim + 1] = l_run;
    }
  }
  __syncthreads();

  for (uint32_t idx = tid; idx < heads_here * kHeadDim; idx += kDecWaves * kWave) {
    const uint32_t h = idx / kHeadDim, d = idx % kHeadDim;
    float mw[kDecWaves];
    float mmax = -INFINITY;
#pragma unroll
    for (int w = 0; w < kDecWaves; ++w) {
      mw[w] = red[(w * kMaxHeadsPerGroup + h) * kRedPitch + kHeadDim];
      mmax = fmaxf(mmax, mw[w]);
    }
    float lsum = 0.0f, a = 0.0f;
#pragma unroll
    for (int w = 0; w < kDecWaves; ++w) {
      const float wgt = (mw[w] == -INFINITY) ? 0.0f : fast_exp2(mw[w] - mmax);
      lsum += wgt * red[(w * kMaxHeadsPerGroup + h) * kRedPitch + kHeadDim + 1];
      a += wgt * red[(w * kMaxHeadsPerGroup + h) * kRedPitch + d];
    }
    const uint32_t head = head0 + h;
    if (p.n_split == 1) {
      const size_t o = ((size_t)seq * p.n_q_heads + head) * kHeadDim + d;
      const float val = a / lsum;
      p.out[o] = (uint16_t)(Mfma<T>::pack2(val, 0.0f) & 0xffffu);
      if (p.lse && d == 0)
        p.lse[(size_t)seq * p.n_q_heads + head] = (mmax + fast_log2(lsum)) * kLn2;
    } else {
      const size_t prow = ((size_t)seq * p.n_q_heads + head) * p.n_split + split;
      p.ws_acc[prow * kHeadDim + d] = a;
      if (d == 0) {
        p.ws_ml[prow * 2] = mmax;
        p.ws_ml[prow * 2 + 1] = lsum;
      }
    }
  }
}

// One workgroup of 128 threads per (sequence, query head): combine the live
// splits' (max, sum, acc) into the normalised output row and its log-sum-exp.
template <typename T>
__global__ __launch_bounds__(kHeadDim) void merge_kernel(DecodeKernelArgs p) {
  const uint32_t row = blockIdx.x;  // seq * n_q_heads + head
  const uint32_t seq = row / p.n_q_heads;
  const uint32_t d = threadIdx.x;
  uint32_t pos = p.position;
  if (p.positions) pos = min(p.positions[seq], p.position);
  const uint32_t live = min(p.n_split, (pos + p.split_len) / p.split_len);  // ceil((pos+1)/split_len)
  const float* ml = p.ws_ml + (size_t)row * p.n_split * 2;
  const float* accp = p.ws_acc + (size_t)row * p.n_split * kHeadDim;
  float mmax = -INFINITY;
  for (uint32_t s = 0; s < live; ++s) mmax = fmaxf(mmax, ml[2 * s]);
  float lsum = 0.0f, a = 0.0f;
  for (uint32_t s = 0; s < live; ++s) {
    const float wgt = fast_exp2(ml[2 * s] - mmax);
    lsum += wgt * ml[2 * s + 1];
    a += wgt * accp[(size_t)s * kHeadDim + d];
  }
  const float val = a / lsum;
  p.out[(size_t)row * kHeadDim + d] = (uint16_t)(Mfma<T>::pack2(val, 0.0f) & 0xffffu);
  if (p.lse && d == 0) p.lse[row] = (mmax + fast_log2(lsum)) * kLn2;
}

}  // namespace

DecodePlan decode_plan(uint32_t max_len, uint32_t batch, uint32_t n_kv_heads, uint32_t n_cu) {
  // Aim for about four resident workgroups per compute unit (the LDS footprint
  // allows four), but never make a split shorter than four 64-key steps.
  const uint32_t target = n_cu * 4;
  const uint32_t planes = batch * n_kv_heads;
  const uint32_t want = (target + planes - 1) / planes;
  uint32_t split_len = (max_len + want - 1) / want;
  split_len = (split_len + kDecodeStepKeys - 1) / kDecodeStepKeys * kDecodeStepKeys;
  if (split_len < 4 * kDecodeStepKeys) split_len = 4 * kDecodeStepKeys;
  DecodePlan plan;
  plan.split_len = split_len;
  plan.n_split = (max_len + split_len - 1) / split_len;
  return plan;
}

size_t decode_workspace_rows(uint32_t batch_capacity, uint32_t n_q_heads, uint32_t n_kv_heads,
                             uint32_t n_cu) {
  // rows = batch * heads * n_split with n_split <= ceil(4*n_cu / (batch*kv_heads))
  const size_t group = n_q_heads / n_kv_heads;
  return (size_t)batch_capacity * n_q_heads + (size_t)n_cu * 4 * group;
}

hipError_t launch_decode(const AttnArgs& a, hipStream_t stream) {
  DecodeKernelArgs p;
  p.q = (const uint16_t*)a.q;
  p.k = (const uint16_t*)a.k;
  p.v = (const uint16_t*)a.v;
  p.out = (uint16_t*)a.out;
  p.lse = a.lse;
  p.positions = a.positions;
  p.ws_acc = a.ws_acc;
  p.ws_ml = a.ws_ml;
  p.kv_stride_seq = a.kv_stride_seq;
  p.kv_stride_head = a.kv_stride_head;
  p.kv_stride_pos = a.kv_stride_pos;
  p.n_q_heads = a.n_q_heads;
  p.n_kv_heads = a.n_kv_heads;
  p.group = a.group;
  p.head_groups = (a.group + kMaxHeadsPerGroup - 1) / kMaxHeadsPerGroup;
  p.position = a.position_index;
  p.split_len = a.split_len;
  p.n_split = a.n_split;
  p.scale_log2 = a.scale * kLog2e;

  dim3 grid(a.n_split, a.n_kv_heads * p.head_groups, a.batch);
  dim3 block(kDecWaves * kWave);
  if (a.dtype == 0)
    hipLaunchKernelGGL(decode_split_kernel<F16>, grid, block, 0, stream, p);
  else
    hipLaunchKernelGGL(decode_split_kernel<BF16>, grid, block, 0, stream, p);
  hipError_t err = hipGetLastError();
  if (err != hipSuccess) return err;
  if (a.n_split > 1) {
    dim3 mgrid(a.batch * a.n_q_heads);
    if (a.dtype == 0)
      hipLaunchKernelGGL(merge_kernel<F16>, mgrid, dim3(kHeadDim), 0, stream, p);
    else
      hipLaunchKernelGGL(merge_kernel<BF16>, mgrid, dim3(kHeadDim), 0, stream, p);
    err = hipGetLastError();
  }
  return err;
}

}  // namespace ellm
