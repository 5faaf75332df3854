// Attention for the shapes the MFMA kernels do not take: any head size up to 256 and binary32
// storage.  The reference's generic leaf (src/kernel/generic/flash_attention.rs:60-89) honours
// whatever `length` and element type its caller hands it, and its operator test runs in f32
// (src/compiler/mul/attention.rs:262-330); every model the reference ships has 128-wide
// binary16 heads, which go to decode.hip / prefill.hip, so this kernel is written for being
// right on one path, not for a roofline: one workgroup per (token, sequence, query head) row,
// the four waves take the row's keys in turns of four, a lane owns elements lane, lane + 64,
// ... of the head, scores are binary32 dot products reduced over the wave, the soft-max runs
// online in binary32 and the waves' partial rows meet in LDS.  Same arguments, masks, position
// rules and log-sum-exp as the other kernels (ellm_attn_run / ellm_attn_run_ragged).
#include "common.hpp"
#include "kernels.hpp"

namespace ellm {
namespace {

constexpr int kMaxHead = 256;            // head sizes up to 4 x 64 lanes
constexpr int kPerLane = kMaxHead / kWave;
constexpr int kKeysPerTurn = 4;          // keys a wave requests together
constexpr int kGenWaves = 4;

struct F32 {};
template <typename E>
struct Elem;
template <>
struct Elem<F16> {
  typedef uint16_t type;
  static __device__ __forceinline__ float load(const type* p) { return Mfma<F16>::to_float(*p); }
  static __device__ __forceinline__ void store(type* p, float v) { *p = (uint16_t)(Mfma<F16>::pack2(v, 0.0f) & 0xffffu); }
};
template <>
struct Elem<BF16> {
  typedef uint16_t type;
  static __device__ __forceinline__ float load(const type* p) { return Mfma<BF16>::to_float(*p); }
  static __device__ __forceinline__ void store(type* p, float v) { *p = (uint16_t)(Mfma<BF16>::pack2(v, 0.0f) & 0xffffu); }
};
template <>
struct Elem<F32> {
  typedef float type;
  static __device__ __forceinline__ float load(const type* p) { return *p; }
  static __device__ __forceinline__ void store(type* p, float v) { *p = v; }
};

struct GeneralArgs {
  const void* q;
  const void* k;
  const void* v;
  void* out;
  float* lse;
  const uint32_t* positions;
  const size_t* seq_offsets;
  const uint32_t* seq_caps;
  size_t kv_stride_seq, kv_stride_head, kv_stride_pos;
  uint32_t batch_pitch, batch, n_q_heads, group, head_size;
  uint32_t position_index;   // start position, or the bound of the per-sequence positions
  float scale;
};

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) v += __shfl_xor(v, m);
  return v;
}

template <typename S>
__global__ __launch_bounds__(kGenWaves* kWave) void attn_general_kernel(GeneralArgs p) {
  typedef typename Elem<S>::type E;
  __shared__ float s_o[kGenWaves][kMaxHead];
  __shared__ float s_m[kGenWaves], s_l[kGenWaves];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const uint32_t hs = p.head_size;
  // blockIdx.x = (token * batch + sequence) * heads + head over the live sequences
  uint32_t r = blockIdx.x;
  const uint32_t head = r % p.n_q_heads;
  r /= p.n_q_heads;
  const uint32_t seq = r % p.batch, tok = r / p.batch;
  uint32_t pos = p.position_index + tok;
  if (p.positions) pos = min(p.positions[seq], p.position_index);   // single-token calls only
  if (p.seq_caps) pos = min(pos, p.seq_caps[seq] - 1);
  const size_t row = ((size_t)tok * p.batch_pitch + seq) * p.n_q_heads + head;
  const E* q = (const E*)p.q + row * hs;
  const size_t plane = seq_plane_offset(p.seq_offsets, p.kv_stride_seq, seq) + (size_t)(head / p.group) * p.kv_stride_head;
  const E* kp = (const E*)p.k + plane;
  const E* vp = (const E*)p.v + plane;

  float qv[kPerLane], o[kPerLane];
#pragma unroll
  for (int i = 0; i < kPerLane; ++i) {
    const uint32_t d = lane + 64 * i;
    qv[i] = d < hs ? Elem<S>::load(q + d) * p.scale : 0.0f;
    o[i] = 0.0f;
  }
  float m = -INFINITY, l = 0.0f;
  // wave w takes keys 16 n + 4 w .. + 3 (wave-uniform bounds: no lane leaves the reductions)
  for (uint32_t j0 = kKeysPerTurn * wave; j0 <= pos; j0 += kKeysPerTurn * kGenWaves) {
    float kk[kKeysPerTurn][kPerLane], vv[kKeysPerTurn][kPerLane];
#pragma unroll
    for (int u = 0; u < kKeysPerTurn; ++u) {
      const uint32_t j = min(j0 + u, pos);   // keys past the row's own position are masked below
#pragma unroll
      for (int i = 0; i < kPerLane; ++i) {
        const uint32_t d = lane + 64 * i;
        kk[u][i] = d < hs ? Elem<S>::load(kp + (size_t)j * p.kv_stride_pos + d) : 0.0f;
        vv[u][i] = d < hs ? Elem<S>::load(vp + (size_t)j * p.kv_stride_pos + d) : 0.0f;
      }
    }
    float s[kKeysPerTurn];
#pragma unroll
    for (int u = 0; u < kKeysPerTurn; ++u) {
      float part = 0.0f;
#pragma unroll
      for (int i = 0; i < kPerLane; ++i) part = __builtin_fmaf(qv[i], kk[u][i], part);
      s[u] = (j0 + u <= pos) ? wave_sum(part) : -INFINITY;
    }
    float m_new = m;
#pragma unroll
    for (int u = 0; u < kKeysPerTurn; ++u) m_new = fmaxf(m_new, s[u]);
    const float alpha = __expf(m - m_new);   // m = -inf on the first turn: exp(-inf) = 0 (m_new is finite: key j0 counts)
    l *= alpha;
#pragma unroll
    for (int i = 0; i < kPerLane; ++i) o[i] *= alpha;
#pragma unroll
    for (int u = 0; u < kKeysPerTurn; ++u) {
      const float w = __expf(s[u] - m_new);  // masked keys: exp(-inf) = 0
      l += w;
#pragma unroll
      for (int i = 0; i < kPerLane; ++i) o[i] = __builtin_fmaf(w, vv[u][i], o[i]);
    }
    m = m_new;
  }
  // the four waves' partial rows meet in LDS (a wave without keys leaves max = -inf, sum = 0)
#pragma unroll
  for (int i = 0; i < kPerLane; ++i) s_o[wave][lane + 64 * i] = o[i];
  if (lane == 0) {
    s_m[wave] = m;
    s_l[wave] = l;
  }
  __syncthreads();
  float top = s_m[0];   // finite: wave 0 holds key 0
#pragma unroll
  for (int w = 1; w < kGenWaves; ++w) top = fmaxf(top, s_m[w]);
  float sum = 0.0f, wgt[kGenWaves];
#pragma unroll
  for (int w = 0; w < kGenWaves; ++w) {
    wgt[w] = __expf(s_m[w] - top);
    sum += wgt[w] * s_l[w];
  }
  const float inv = 1.0f / sum;
  E* out = (E*)p.out + row * hs;
  for (uint32_t d = threadIdx.x; d < hs; d += blockDim.x) {
    float acc = 0.0f;
#pragma unroll
    for (int w = 0; w < kGenWaves; ++w) acc += wgt[w] * s_o[w][d];
    Elem<S>::store(out + d, acc * inv);
  }
  if (p.lse && threadIdx.x == 0) p.lse[row] = top + __logf(sum);
}

}  // namespace

hipError_t launch_attn_general(const AttnArgs& a, uint32_t head_size, hipStream_t stream) {
  GeneralArgs p;
  p.q = a.q;
  p.k = a.k;
  p.v = a.v;
  p.out = a.out;
  p.lse = a.lse;
  p.positions = a.positions;
  p.seq_offsets = a.seq_offsets;
  p.seq_caps = a.seq_caps;
  p.kv_stride_seq = a.kv_stride_seq;
  p.kv_stride_head = a.kv_stride_head;
  p.kv_stride_pos = a.kv_stride_pos;
  p.batch_pitch = a.batch_pitch;
  p.batch = a.batch;
  p.n_q_heads = a.n_q_heads;
  p.group = a.group;
  p.head_size = head_size;
  p.position_index = a.position_index;
  p.scale = a.scale;
  const size_t rows = (size_t)a.position_interval * a.batch * a.n_q_heads;
  if (rows == 0) return hipSuccess;
  if (rows > 0x7fffffffu || head_size == 0 || head_size > (uint32_t)kMaxHead) return hipErrorInvalidValue;
  const dim3 grid((uint32_t)rows), block(kGenWaves * kWave);
  if (a.dtype == 0)
    hipLaunchKernelGGL(attn_general_kernel<F16>, grid, block, 0, stream, p);
  else if (a.dtype == 1)
    hipLaunchKernelGGL(attn_general_kernel<BF16>, grid, block, 0, stream, p);
  else
    hipLaunchKernelGGL(attn_general_kernel<F32>, grid, block, 0, stream, p);
  return hipGetLastError();
}

}  // namespace ellm
