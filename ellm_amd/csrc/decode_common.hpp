// Building blocks of the single-token attention kernels (decode.hip: one position range for
// every workgroup of a plane; decode_balanced.hip: per-sequence lengths dealt evenly over the
// workgroups): the per-wave key stream, the merge of a workgroup's four waves, the arrival
// count and the fold of partial results.
#pragma once

#include "common.hpp"
#include "kernels.hpp"

namespace ellm {
namespace dec {

constexpr int kDecWaves = 4;
constexpr int kDecThreads = kDecWaves * kWave;
constexpr int kChunk = 16;                      // keys per wave step
constexpr int kKPitch = kHeadDim + 8;           // halves per K row in LDS (272 B)
constexpr int kVtPitch = kChunk + 4;            // halves per V^T row in LDS (40 B)
constexpr int kWaveLdsHalves = kChunk * kKPitch + kHeadDim * kVtPitch;
constexpr int kMaxHeadsPerGroup = 16;
static_assert(kMaxHeadsPerGroup == (int)kPlanMaxHeadsPerGroup, "decode_plan.hpp sizes the workspace for this group");
constexpr int kMergeFan = 16;                   // partials folded per merge step
static_assert(kMergeFan == (int)kPlanMergeFan, "decode_plan.hpp sizes the workspace for this fan");
constexpr int kQuads = kHeadDim / 4;
constexpr int kItems = kMaxHeadsPerGroup * kQuads / kDecThreads;  // (head, four columns) items per thread
constexpr int kRedPitch = kHeadDim + 4;         // floats per (wave, head) row of the wave merge, 16-byte aligned
static_assert(kDecWaves * kMaxHeadsPerGroup * kRedPitch * 4 <= kDecWaves * kWaveLdsHalves * 2,
              "reduction buffer must fit in the staging buffers");

struct DecodeKernelArgs {
  const uint16_t* q;
  const uint16_t* k;
  const uint16_t* v;
  uint16_t* out;
  float* lse;
  const uint32_t* positions;
  const size_t* seq_offsets;   // per-sequence plane offsets (null: sequence x kv_stride_seq)
  const uint32_t* seq_caps;    // per-sequence capacities (null: none to clamp to)
  float* ws_acc;
  float* ws_ml;
  float* ws2_acc;      // cluster partials
  float* ws2_ml;
  uint32_t* counters;  // arrival counters; all zero between launches
  uint32_t counters_per_plane, n_cluster_max;
  size_t kv_stride_seq, kv_stride_head, kv_stride_pos;
  uint32_t n_q_heads, n_kv_heads, group, head_groups;
  uint32_t position;  // shared position (positions == null) or upper bound
  uint32_t split_len, n_split;
  uint32_t batch;     // sequences (decode_balanced.hip)
  uint32_t wgs_one;   // workgroups that find a compute unit each (decode_balanced.hip)
  float scale_log2;   // scale * log2(e)
  PendingRows pend;   // raw query / key / value rows of a fused step (kernels built with PENDING)
};

// Agent-scope (device-wide coherent) relaxed 8-byte load / store of a pair of floats.
__device__ __forceinline__ uint64_t load_coherent64(const float* p) {
  return __hip_atomic_load((const uint64_t*)p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void store_coherent64(float* p, float lo, float hi) {
  const uint64_t bits = (uint64_t)__builtin_bit_cast(uint32_t, lo) |
                        ((uint64_t)__builtin_bit_cast(uint32_t, hi) << 32);
  __hip_atomic_store((uint64_t*)p, bits, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// Agent-scope load of four floats at byte offset `off` of a table: a buffer load with the
// sc1 cache-policy bit (what the compiler's own agent-scope atomic loads carry).  There is no
// 16-byte atomic load; as a builtin the compiler tracks the load's completion itself.
constexpr int kCachePolicySc1 = 16;
__device__ __forceinline__ f32x4 load_coherent128(__amdgpu_buffer_rsrc_t table, uint32_t off) {
  return __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(table, off, 0, kCachePolicySc1));
}
__device__ __forceinline__ __amdgpu_buffer_rsrc_t table_rsrc(const float* table) {
  return __builtin_amdgcn_make_buffer_rsrc((void*)table, 0, 0xffffffffu, 0x00020000);
}
// Block until every vector-memory operation this wave has issued is complete
// (s_waitcnt vmcnt(0); expcnt and lgkmcnt left at their maxima).
__device__ __forceinline__ void wait_vm_done() { __builtin_amdgcn_s_waitcnt(0x0F70); }

// K/V rows are read once and never reused: non-temporal loads (measured 8 % faster)
__device__ __forceinline__ u32x4 stream_load16(const uint16_t* p) {
  return __builtin_nontemporal_load((const u32x4*)p);
}

// What a thread is inside its workgroup of four waves.
struct Lane {
  int tid, wave, lane;
  int g, c;  // lane / 16, lane % 16
  __device__ __forceinline__ Lane() {
    tid = threadIdx.x;
    wave = tid >> 6;
    lane = tid & 63;
    g = lane >> 4;
    c = lane & 15;
  }
};

// Query heads of a group as the B operand of S^T = K.Q^T: lane (head c, group g) holds
// q[head][32 s + 8 g + 0..7] for s = 0..3; heads past the group's end are zero.
__device__ __forceinline__ void load_queries(const uint16_t* q_rows, const Lane& t, uint32_t heads_here,
                                             u32x4 (&qreg)[4]) {
  const uint16_t* qrow = q_rows + (size_t)t.c * kHeadDim;
#pragma unroll
  for (int s = 0; s < 4; ++s) {
    if ((uint32_t)t.c < heads_here)
      qreg[s] = load16(qrow + 32 * s + 8 * t.g);
    else
      qreg[s] = u32x4{0, 0, 0, 0};
  }
}

// ---- fused step: the rows the projection left raw ----------------------------------------

// Eight consecutive raw values: binary32 partial sums, one or two of them `stride` floats apart.
// Fetched first (two or four 16-byte loads, nothing waits) and added up later, so that the
// caller can put other loads in flight between the two.
struct Raw8 {
  f32x4 lo[2], hi[2];
  __device__ __forceinline__ void fetch(const float* src, uint32_t parts, uint32_t stride) {
    lo[0] = *(const f32x4*)src;
    hi[0] = *(const f32x4*)(src + 4);
    lo[1] = hi[1] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    if (parts > 1) {   // (uniform)
      lo[1] = *(const f32x4*)(src + stride);
      hi[1] = *(const f32x4*)(src + stride + 4);
    }
  }
  __device__ __forceinline__ void sum(float (&x)[8]) const {
    const f32x4 l = lo[0] + lo[1], h = hi[0] + hi[1];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      x[e] = l[e];
      x[4 + e] = h[e];
    }
  }
};

// load_queries() for a fused step: the group's query rows come as raw sums and are normalised
// and rotated on the way into the operand registers.  Lane (head c, group g) holds the octets
// 4 s + g of its head; the sum of squares is added up in the order the projection's own
// finishing step uses (octet, pairs of octets, fours, eights, all sixteen), so the rows come
// out with the bits that step gives them.
struct PendingQueries {
  Raw8 raw[4];
  u32x4 rope[4];
  __device__ __forceinline__ void fetch(const PendingRows& pr, uint32_t seq, uint32_t head0, uint32_t pos,
                                        const Lane& t, uint32_t heads_here) {
    const uint32_t head = head0 + ((uint32_t)t.c < heads_here ? t.c : 0);
    const float* src = pr.raw + (size_t)seq * pr.cols + (size_t)head * kHeadDim + 8 * t.g;
    const uint16_t* row = (const uint16_t*)pr.rope + (size_t)pos * pr.rope_pos_stride +
                          (size_t)head * pr.rope_head_stride + 8 * t.g;
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      raw[s].fetch(src + 32 * s, pr.parts, pr.part_stride);
      rope[s] = load16(row + 32 * s);
    }
  }
  template <typename T>
  __device__ __forceinline__ void finish(float eps, const Lane& t, uint32_t heads_here, u32x4 (&qreg)[4]) const {
    float x[4][8], ss[4];
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      raw[s].sum(x[s]);
      ss[s] = squares8(x[s]);
    }
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      ss[s] += xor_shuffle(ss[s], 16);
      ss[s] += xor_shuffle(ss[s], 32);
    }
    const float inv = inverse_rms((ss[0] + ss[1]) + (ss[2] + ss[3]), eps);
    const bool live = (uint32_t)t.c < heads_here;
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      qreg[s] = scale_rotate_pack8<T>(x[s], inv, rope[s]);
      if (!live) qreg[s] = u32x4{0, 0, 0, 0};
    }
  }
};
// The finished query rows go back to where the projection alone would have left them.
__device__ __forceinline__ void store_queries(uint16_t* q_rows, const Lane& t, uint32_t heads_here,
                                              const u32x4 (&qreg)[4]) {
  if ((uint32_t)t.c >= heads_here) return;
#pragma unroll
  for (int s = 0; s < 4; ++s) store16(q_rows + (size_t)t.c * kHeadDim + 32 * s + 8 * t.g, qreg[s]);
}

// The key and value row a fused step adds to a plane: where their raw sums are, and the cache
// rows they belong in (written by the workgroup that holds the plane's last key).
struct NewRow {
  bool present;              // this stretch of keys ends with the plane's new key
  bool store;                // ... and this workgroup is the one that writes it to the cache
  const float* k_raw;        // kPendSums: 128 raw sums each (first part)
  const float* v_raw;
  uint32_t parts, part_stride;
  const uint16_t* k_row16;   // kPendRows: the 128-element source rows
  const uint16_t* v_row16;
  const uint16_t* rope_row;  // rotary row of (position, kv head)
  float eps;
  uint16_t* k_dst;
  uint16_t* v_dst;
};
// What a launch finds pending (template argument of the kernels and of stream_keys).
constexpr int kPendNone = 0;   // the ordinary launch
constexpr int kPendSums = 1;   // a fused projection step: raw binary32 sums of the query, key and value rows
constexpr int kPendRows = 2;   // a fused cache write: stored 16-bit key / value rows, queries final

// The new row of plane (sequence, kv head) at position pos, as the launch's PendingRows describe it.
template <int MODE>
__device__ __forceinline__ NewRow new_row_of(const PendingRows& pr, uint32_t seq, uint32_t kvh, uint32_t pos,
                                             uint32_t n_q_heads, uint32_t n_kv_heads, uint16_t* k_dst, uint16_t* v_dst,
                                             bool present, bool store) {
  NewRow n;
  n.present = present;
  n.store = store;
  n.k_raw = n.v_raw = nullptr;
  n.parts = n.part_stride = 0;
  n.k_row16 = n.v_row16 = nullptr;
  if constexpr (MODE == kPendSums) {
    const size_t col_k = (size_t)seq * pr.cols + (size_t)(n_q_heads + kvh) * kHeadDim;
    n.k_raw = pr.raw + col_k;
    n.v_raw = pr.raw + col_k + (size_t)n_kv_heads * kHeadDim;
    n.parts = pr.parts;
    n.part_stride = pr.part_stride;
  } else {
    const size_t row = ((size_t)seq * n_kv_heads + kvh) * kHeadDim;
    n.k_row16 = (const uint16_t*)pr.k_rows + row;
    n.v_row16 = (const uint16_t*)pr.v_rows + row;
  }
  n.rope_row = (const uint16_t*)pr.rope + (size_t)pos * pr.rope_pos_stride + (size_t)kvh * pr.rope_head_stride;
  n.eps = pr.eps;
  n.k_dst = k_dst;
  n.v_dst = v_dst;
  return n;
}
// Every lane c of each 16-lane group ends up with elements 8 c .. 8 c + 7 of the finished rows
// (the arithmetic of the projection's own finishing step, lane for lane).
template <int MODE>
struct NewRowLoads;
template <>
struct NewRowLoads<kPendSums> {
  Raw8 k, v;
  u32x4 rope;
  __device__ __forceinline__ void fetch(const NewRow& n, const Lane& t) {
    k.fetch(n.k_raw + 8 * t.c, n.parts, n.part_stride);
    v.fetch(n.v_raw + 8 * t.c, n.parts, n.part_stride);
    rope = load16(n.rope_row + 8 * t.c);
  }
  template <typename T>
  __device__ __forceinline__ void finish(const NewRow& n, const Lane& t, u32x4& knew, u32x4& vnew) const {
    float kx[8], vx[8];
    k.sum(kx);
    v.sum(vx);
    float ss = squares8(kx);
#pragma unroll
    for (int m = 1; m < 16; m <<= 1) ss += __shfl_xor(ss, m, 16);
    knew = scale_rotate_pack8<T>(kx, inverse_rms(ss, n.eps), rope);
    vnew = u32x4{Mfma<T>::pack2(vx[0], vx[1]), Mfma<T>::pack2(vx[2], vx[3]), Mfma<T>::pack2(vx[4], vx[5]),
                 Mfma<T>::pack2(vx[6], vx[7])};
    if (n.store && t.g == 0) {
      store16(n.k_dst + 8 * t.c, knew);
      store16(n.v_dst + 8 * t.c, vnew);
    }
  }
};
// Stored 16-bit rows: the cache write's own arithmetic (norm_rope_row16), so the row that lands in
// the cache carries the bits ellm_kv_append_norm_rope would have written.
template <>
struct NewRowLoads<kPendRows> {
  u32x4 k, v, rope;
  __device__ __forceinline__ void fetch(const NewRow& n, const Lane& t) {
    k = load16(n.k_row16 + 8 * t.c);
    v = load16(n.v_row16 + 8 * t.c);
    rope = load16(n.rope_row + 8 * t.c);
  }
  template <typename T>
  __device__ __forceinline__ void finish(const NewRow& n, const Lane& t, u32x4& knew, u32x4& vnew) const {
    knew = norm_rope_row16<T>(k, rope, n.eps);
    vnew = v;
    if (n.store && t.g == 0) {
      store16(n.k_dst + 8 * t.c, knew);
      store16(n.v_dst + 8 * t.c, vnew);
    }
  }
};
template <>
struct NewRowLoads<kPendNone> {
  __device__ __forceinline__ void fetch(const NewRow&, const Lane&) {}
  template <typename T>
  __device__ __forceinline__ void finish(const NewRow&, const Lane&, u32x4&, u32x4&) const {}
};

// One wave's share of keys [k_begin, k_end) of a plane: the four waves take alternating 16-key
// chunks, each streams its chunks HBM -> registers (128-bit loads, four full 256-byte rows per
// instruction) -> its private LDS slice -> MFMA operands, so no workgroup barrier is needed
// inside the loop.  Scores S^T[key][head] = K.Q^T on 16x16x32 MFMA with up to 16 query heads in
// the N dimension; O^T[d][head] += V^T.P^T on 16x16x16 MFMA, whose B-operand layout is exactly
// the C layout S^T comes out in.  V is transposed on the way into LDS with 4-key x 8-dim
// register blocks.  Leaves the wave's running maximum (log2 units), this lane's share of the
// denominator summed over its partner lanes, and the unnormalised output columns.
// Chunks are visited in an order rotated by `rot_seed` (soft-max accumulation does not care
// about order): splits start at offsets that are multiples of the split length, and walking
// them in lockstep would keep every stream on the same few HBM channels.
// PENDING (a fused step): when `fresh.present`, key `pos` is not in the cache yet; the stream
// covers [k_begin, pos) and the wave with the fewest chunks finishes the new key / value row
// from the projection's raw sums (requested before its stream starts), writes it to the cache
// and takes it as one more chunk of its own.
// The raw rows are requested ahead of the wave's first chunk of keys and finished behind its
// request (`queries` holds the requested raw query rows; qreg is filled here), so that both
// trips to memory run side by side.  With kPendRows (a fused cache write) the new rows come as
// stored 16-bit rows, the query rows are final (qreg filled by the caller, `queries` null).
template <typename T, int PENDING = kPendNone>
__device__ __forceinline__ void stream_keys(const uint16_t* kplane, const uint16_t* vplane, size_t stride_pos,
                                            uint32_t k_begin, uint32_t k_end, uint32_t pos,
                                            u32x4 (&qreg)[4], uint16_t* smem, const Lane& t,
                                            uint32_t rot_seed, float scale_log2, float& m_out, float& l_out,
                                            f32x4 (&acc)[8], const NewRow* fresh = nullptr,
                                            const PendingQueries* queries = nullptr, uint32_t heads_here = 0) {
  const int g = t.g, c = t.c, wave = t.wave;
  uint16_t* ks = smem + wave * kWaveLdsHalves;  // [16][kKPitch]
  uint16_t* vt = ks + kChunk * kKPitch;         // [128][kVtPitch]

  const uint32_t new_pos = pos;   // (PENDING) the position of the new key
  bool take_new = false;
  if constexpr (PENDING) {
    if (fresh->present) {   // the stream ends before the new key; its last valid row is pos - 1
      k_end = pos;
      pos = pos ? pos - 1 : 0;
    }
  }
  const uint32_t n_chunks = (k_end - k_begin + kChunk - 1) / kChunk;
  u32x4 knew = {0, 0, 0, 0}, vnew = {0, 0, 0, 0};
  if constexpr (PENDING) take_new = fresh->present && (uint32_t)wave == n_chunks % kDecWaves;   // (uniform over the wave)
  // one 16-key chunk in flight per wave (a second one measured no faster)
  u32x4 kreg[4], vreg[4];
  auto issue_loads = [&](uint32_t chunk) {
    const uint32_t kb = k_begin + chunk * kChunk;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      // rows past the last valid key are clamped onto it: always in bounds,
      // always initialised, and their probabilities are forced to zero below.
      const uint32_t row = min(kb + 4 * g + i, pos);
      kreg[i] = stream_load16(kplane + (size_t)row * stride_pos + 8 * c);
      vreg[i] = stream_load16(vplane + (size_t)row * stride_pos + 8 * c);
    }
  };

  float m_run = -INFINITY;  // running max, log2 units (score * scale * log2 e)
  float l_run = 0.0f;       // this lane's share of the denominator
#pragma unroll
  for (int b = 0; b < 8; ++b) acc[b] = f32x4{0, 0, 0, 0};

  const uint32_t my_chunks = (n_chunks > (uint32_t)wave) ? (n_chunks - wave + kDecWaves - 1) / kDecWaves : 0;
  const uint32_t rot = rot_seed % max(my_chunks, 1u);
  auto chunk_at = [&](uint32_t it) {
    uint32_t r = it + rot;
    if (r >= my_chunks) r -= my_chunks;
    return wave + r * kDecWaves;
  };
  // registers -> LDS: K row-major, V transposed.
  auto stage = [&]() {
#pragma unroll
    for (int i = 0; i < 4; ++i) store16(ks + (4 * g + i) * kKPitch + 8 * c, kreg[i]);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      u32x2 col = gather_column(vreg[0][e >> 1], vreg[1][e >> 1], vreg[2][e >> 1],
                                vreg[3][e >> 1], (e & 1) != 0);
      *(u32x2*)(vt + (8 * c + e) * kVtPitch + 4 * g) = col;
    }
  };
  // the staged chunk, keys kb .. kb + 15 of which those up to `last` count
  auto consume = [&](uint32_t kb, uint32_t last) {
    // S^T[key][head], lane (head c, group g) register r <-> key kb + 4 g + r.
    f32x4 st = {0, 0, 0, 0};
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      u32x4 a = load16(ks + c * kKPitch + 32 * s + 8 * g);
      st = Mfma<T>::m16x16x32(a, qreg[s], st);
    }
    float tt[4];
    float tmax = -INFINITY;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      tt[r] = (kb + 4 * g + r <= last) ? st[r] * scale_log2 : -INFINITY;
      tmax = fmaxf(tmax, tt[r]);
    }
    tmax = fmaxf(tmax, xor_shuffle(tmax, 16));
    tmax = fmaxf(tmax, xor_shuffle(tmax, 32));
    const float m_new = fmaxf(m_run, tmax);  // finite: key kb is always valid
    const float alpha = fast_exp2(m_run - m_new);
    float pr[4];
    float psum = 0.0f;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      pr[r] = fast_exp2(tt[r] - m_new);
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
  };

  NewRowLoads<PENDING> fresh_loads;
  if constexpr (PENDING) {
    if (take_new) fresh_loads.fetch(*fresh, t);
  }
  if (my_chunks) issue_loads(chunk_at(0));
  if constexpr (PENDING == kPendSums) queries->template finish<T>(fresh->eps, t, heads_here, qreg);
  if constexpr (PENDING) {
    if (take_new) fresh_loads.template finish<T>(*fresh, t, knew, vnew);   // (the whole wave: uniform)
  }
  for (uint32_t it = 0; it < my_chunks; ++it) {
    const uint32_t chunk = chunk_at(it);
    const uint32_t kb = k_begin + chunk * kChunk;
    stage();
    if (it + 1 < my_chunks) issue_loads(chunk_at(it + 1));
    __builtin_amdgcn_wave_barrier();
    consume(kb, pos);
    __builtin_amdgcn_wave_barrier();
  }
  if constexpr (PENDING) {
    if (take_new) {   // a chunk whose first row is the new key; its other rows are zeros and do not count
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const bool first = g == 0 && i == 0;
        kreg[i] = first ? knew : u32x4{0, 0, 0, 0};
        vreg[i] = first ? vnew : u32x4{0, 0, 0, 0};
      }
      stage();
      __builtin_amdgcn_wave_barrier();
      consume(new_pos, new_pos);
      __builtin_amdgcn_wave_barrier();
    }
  }

  l_run += xor_shuffle(l_run, 16);
  l_run += xor_shuffle(l_run, 32);
  m_out = m_run;
  l_out = l_run;
}

// Merge the four waves through LDS (red[wave][head][128 acc + max + sum], in the staging
// buffers).  Afterwards a thread owns four consecutive columns of one head (an item; eight heads
// make 256 items, one per thread, sixteen heads two per thread) and hands them to
// emit(h, dq, a[4], sum, max): columns 4 dq .. 4 dq + 3 of head h of the group.
template <typename Emit>
__device__ __forceinline__ void merge_waves(uint16_t* smem, const Lane& t, uint32_t heads_here, float m_run,
                                            float l_run, const f32x4 (&acc)[8], Emit emit) {
  __syncthreads();
  float* red = (float*)smem;
  if ((uint32_t)t.c < heads_here) {
    float* row = red + (t.wave * kMaxHeadsPerGroup + t.c) * kRedPitch;
#pragma unroll
    for (int b = 0; b < 8; ++b) *(f32x4*)(row + 16 * b + 4 * t.g) = acc[b];
    if (t.g == 0) *(f32x2*)(row + kHeadDim) = f32x2{m_run, l_run};
  }
  __syncthreads();
  const uint32_t n_items = heads_here * kQuads;
#pragma unroll
  for (int n = 0; n < kItems; ++n) {
    const uint32_t item = t.tid + n * kDecThreads;
    if (item >= n_items) continue;
    const uint32_t h = item / kQuads, dq = item % kQuads;
    f32x2 ml[kDecWaves];
    f32x4 part[kDecWaves];
#pragma unroll
    for (int w = 0; w < kDecWaves; ++w) {
      const float* row = red + (w * kMaxHeadsPerGroup + h) * kRedPitch;
      ml[w] = *(const f32x2*)(row + kHeadDim);
      part[w] = *(const f32x4*)(row + 4 * dq);
    }
    float mmax = -INFINITY;
#pragma unroll
    for (int w = 0; w < kDecWaves; ++w) mmax = fmaxf(mmax, ml[w][0]);
    float lsum = 0.0f;
    f32x4 a = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int w = 0; w < kDecWaves; ++w) {
      const float wgt = (ml[w][0] == -INFINITY) ? 0.0f : fast_exp2(ml[w][0] - mmax);
      lsum += wgt * ml[w][1];
      a += wgt * part[w];
    }
    emit(h, dq, a, lsum, mmax);
  }
}

// Columns 4 dq .. of output row `row` (sequence x query heads + head), normalised; the row's
// log-sum-exp with them when asked for.
template <typename T>
__device__ __forceinline__ void emit_final(uint16_t* out, float* lse, size_t row, uint32_t dq, const f32x4& a,
                                           float l, float m) {
  const float inv = 1.0f / l;
  u32x2 w;
  w[0] = Mfma<T>::pack2(a[0] * inv, a[1] * inv);
  w[1] = Mfma<T>::pack2(a[2] * inv, a[3] * inv);
  *(u32x2*)(out + row * kHeadDim + 4 * dq) = w;
  if (lse && dq == 0) lse[row] = (m + fast_log2(l)) * kLn2;
}

// Partial row `prow` of a table of partials: columns 4 dq .. and, once per row, (max, sum).
__device__ __forceinline__ void store_partial(float* acc_tab, float* ml_tab, size_t prow, uint32_t dq,
                                              const f32x4& a, float l, float m) {
  store_coherent64(acc_tab + prow * kHeadDim + 4 * dq, a[0], a[1]);
  store_coherent64(acc_tab + prow * kHeadDim + 4 * dq + 2, a[2], a[3]);
  if (dq == 0) store_coherent64(ml_tab + prow * 2, m, l);
}

// Partials are written and read with agent-scope atomic accesses, which go through to the
// device-wide point of coherence on their own (each XCD has its own L2), so no cache write-back
// or invalidate is needed: a device-scope fence costs a whole-L2 operation per wave and, with a
// thousand workgroups, several times the kernel itself.  Ordering is explicit instead: every
// thread waits until its own partial stores have been acknowledged, the workgroup barrier
// collects all of them, and only then is the arrival counted; the merging workgroup issues its
// loads only after the counter's return value has been seen by all of its threads.
// Returns true in the workgroup that arrives last of `expected`; that one also puts the counter
// back to zero for the next launch (nobody else touches it in this one).
__device__ __forceinline__ bool arrive(uint32_t* counter, uint32_t expected, uint32_t* s_last, int tid) {
  wait_vm_done();
  __syncthreads();
  if (tid == 0) {
    const uint32_t old = __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const uint32_t last = (old + 1 == expected) ? 1u : 0u;
    if (last) __hip_atomic_store(counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    *s_last = last;
  }
  __syncthreads();
  return *s_last != 0;
}

// Fold `count` (<= 16) partials of every head of a group.  Partial i of head h is row
// base_row + h * head_stride + i * part_stride of the tables.  A thread issues every load its
// item needs before it uses any: a fold costs one trip to memory, an 8-byte (max, sum) pair per
// thread, shared through LDS, and one 16-byte accumulator quad per partial; the pairs come back
// from LDS into registers in one go as well (read one by one inside the loops below, every LDS
// round trip showed: 1.1 us for eight partials).  emit(h, dq, a[4], sum, max) receives columns
// 4 dq .. 4 dq + 3.  (The tables stay far below 4 GB: rows and byte offsets fit 32 bits.)
template <typename Emit>
__device__ __forceinline__ void fold(uint16_t* smem, const Lane& t, uint32_t heads_here, const float* acc_tab,
                                     const float* ml_tab, uint32_t base_row, uint32_t head_stride,
                                     uint32_t part_stride, uint32_t count, Emit emit) {
  float* sm = (float*)smem;  // [head][kMergeFan][2]; the reduction buffer is idle by now
  const __amdgpu_buffer_rsrc_t acc_rsrc = table_rsrc(acc_tab);
  const uint32_t n_items = heads_here * kQuads;
  const uint32_t n_ml = heads_here * count;
  const uint32_t h_e = t.tid / count, s_e = t.tid % count;
  uint64_t ml_bits = 0;
  if ((uint32_t)t.tid < n_ml)
    ml_bits = load_coherent64(ml_tab + (size_t)(base_row + h_e * head_stride + s_e * part_stride) * 2);
#pragma unroll
  for (int n = 0; n < kItems; ++n) {
    const uint32_t item = t.tid + n * kDecThreads;
    const bool mine = item < n_items;
    const uint32_t h = mine ? item / kQuads : 0, dq = item % kQuads;
    const uint32_t at = ((base_row + h * head_stride) * kHeadDim + 4 * dq) * 4;
    const uint32_t step = part_stride * kHeadDim * 4;
    f32x4 av[kMergeFan];
#pragma unroll
    for (int i = 0; i < kMergeFan; ++i) {
      av[i] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
      if (mine && (uint32_t)i < count) av[i] = load_coherent128(acc_rsrc, at + (uint32_t)i * step);
    }
    if (n == 0) {  // (every thread passes here once: the branch holds a barrier)
      if ((uint32_t)t.tid < n_ml) *(uint64_t*)(sm + (h_e * kMergeFan + s_e) * 2) = ml_bits;
      __syncthreads();
    }
    if (!mine) continue;
    const float* hm = sm + h * kMergeFan * 2;
    f32x2 ml[kMergeFan];
#pragma unroll
    for (int i = 0; i < kMergeFan; ++i)
      ml[i] = (uint32_t)i < count ? *(const f32x2*)(hm + 2 * i) : f32x2{-INFINITY, 0.0f};
    float m_new = ml[0][0];
#pragma unroll
    for (int i = 1; i < kMergeFan; ++i) m_new = fmaxf(m_new, ml[i][0]);
    float l_acc = 0.0f;
    f32x4 a = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int i = 0; i < kMergeFan; ++i) {
      const float wgt = fast_exp2(ml[i][0] - m_new);  // (an absent entry weighs exp2(-inf) = 0)
      l_acc += wgt * ml[i][1];
      a += wgt * av[i];
    }
    emit(h, dq, a, l_acc, m_new);
  }
}

}  // namespace dec
}  // namespace ellm
