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
//   the partial (max, sum, acc[128]) goes to the workspace, and the workgroup
//   that finishes last for a (sequence, head group) combines that group's
//   splits (a self-resetting arrival counter per group; no second launch).

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
constexpr int kMergeFan = 16;                   // partials folded per merge step

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
  float* ws2_acc;      // cluster partials [sequence][query head][n_cluster_max][128]
  float* ws2_ml;
  uint32_t* counters;  // per (sequence, kv head, head group): [0] clusters done, [1 + c] splits of
                       // cluster c done; all zero between launches
  uint32_t counters_per_plane, n_cluster_max;
  size_t kv_stride_seq, kv_stride_head, kv_stride_pos;
  uint32_t n_q_heads, n_kv_heads, group, head_groups;
  uint32_t position;  // shared position (positions == null) or upper bound
  uint32_t split_len, n_split;
  float scale_log2;   // scale * log2(e)
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

template <typename T>
__global__ __launch_bounds__(kDecWaves* kWave, 4) void decode_split_kernel(
    DecodeKernelArgs p) {
  __shared__ __attribute__((aligned(16))) uint16_t smem[kDecWaves * kWaveLdsHalves];

  // The split a workgroup takes is rotated by its plane's number.  Workgroups are dealt to the
  // eight XCDs by their linear id; with the unrotated mapping (and a split count that is a
  // multiple of 8) one XCD would read the same stretch of every plane, and XCDs differ in how
  // fast they reach a given stretch of memory: 4 sequences x 32768 keys took 51.4 us
  // unrotated, 48.0 us rotated (16 x 8192: no difference).
  const uint32_t split = (blockIdx.x + blockIdx.y + gridDim.y * blockIdx.z) % gridDim.x;
  const uint32_t kvh = blockIdx.y / p.head_groups;
  const uint32_t hgrp = blockIdx.y % p.head_groups;
  const uint32_t seq = blockIdx.z;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int g = lane >> 4, c = lane & 15;

  uint32_t pos = p.position;
  if (p.positions) pos = min(p.positions[seq], p.position);
  if (p.seq_caps) pos = min(pos, p.seq_caps[seq] - 1);
  const uint32_t len = pos + 1;
  const uint32_t k_begin = split * p.split_len;
  const uint32_t k_end = min(len, k_begin + p.split_len);
  const uint32_t heads_here = min((uint32_t)kMaxHeadsPerGroup, p.group - hgrp * kMaxHeadsPerGroup);
  // A split that starts beyond this sequence's keys has nothing to add and is
  // not counted: the merge below derives the live split count from the length.
  if (k_begin >= len) return;

  const size_t plane = seq_plane_offset(p.seq_offsets, p.kv_stride_seq, seq) + kvh * p.kv_stride_head;
  const uint16_t* kplane = p.k + plane;
  const uint16_t* vplane = p.v + plane;

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
  // one 16-key chunk in flight per wave (a second one measured no faster)
  u32x4 kreg[4], vreg[4];
  auto issue_loads = [&](uint32_t chunk) {
    const uint32_t kb = k_begin + chunk * kChunk;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      // rows past the last valid key are clamped onto it: always in bounds,
      // always initialised, and their probabilities are forced to zero below.
      const uint32_t row = min(kb + 4 * g + i, pos);
      kreg[i] = stream_load16(kplane + (size_t)row * p.kv_stride_pos + 8 * c);
      vreg[i] = stream_load16(vplane + (size_t)row * p.kv_stride_pos + 8 * c);
    }
  };

  float m_run = -INFINITY;  // running max, log2 units (score * scale * log2 e)
  float l_run = 0.0f;       // this lane's share of the denominator
  f32x4 acc[8];
#pragma unroll
  for (int b = 0; b < 8; ++b) acc[b] = f32x4{0, 0, 0, 0};

  // Chunks are visited in a rotated order that differs from workgroup to
  // workgroup (soft-max accumulation does not care about order): all splits
  // start at offsets that are multiples of split_len, and walking them in
  // lockstep would keep every stream on the same few HBM channels.
  const uint32_t my_chunks = (n_chunks > (uint32_t)wave) ? (n_chunks - wave + kDecWaves - 1) / kDecWaves : 0;
  const uint32_t rot = (split * 7u + blockIdx.y * 3u + seq * 5u) % max(my_chunks, 1u);
  auto chunk_at = [&](uint32_t it) {
    uint32_t r = it + rot;
    if (r >= my_chunks) r -= my_chunks;
    return wave + r * kDecWaves;
  };
  if (my_chunks) issue_loads(chunk_at(0));
  for (uint32_t it = 0; it < my_chunks; ++it) {
    const uint32_t chunk = chunk_at(it);
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
    if (it + 1 < my_chunks) issue_loads(chunk_at(it + 1));
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
  constexpr int kRedPitch = kHeadDim + 4;  // rows 16-byte aligned
  static_assert(kDecWaves * kMaxHeadsPerGroup * kRedPitch * 4 <= kDecWaves * kWaveLdsHalves * 2,
                "reduction buffer must fit in the staging buffers");
  if ((uint32_t)c < heads_here) {
    float* row = red + (wave * kMaxHeadsPerGroup + c) * kRedPitch;
#pragma unroll
    for (int b = 0; b < 8; ++b) *(f32x4*)(row + 16 * b + 4 * g) = acc[b];
    if (g == 0) *(f32x2*)(row + kHeadDim) = f32x2{m_run, l_run};
  }
  __syncthreads();

  // From here to the end a thread owns four consecutive columns of one head (an item;
  // eight heads make 256 items, one per thread, sixteen heads two per thread).
  constexpr int kQuads = kHeadDim / 4;
  constexpr int kThreads = kDecWaves * kWave;
  constexpr int kItems = kMaxHeadsPerGroup * kQuads / kThreads;
  const uint32_t n_items = heads_here * kQuads;
  auto emit_final = [&](uint32_t h, uint32_t dq, const f32x4& a, float l, float m) {
    const size_t row = (size_t)seq * p.n_q_heads + head0 + h;
    const float inv = 1.0f / l;
    u32x2 w;
    w[0] = Mfma<T>::pack2(a[0] * inv, a[1] * inv);
    w[1] = Mfma<T>::pack2(a[2] * inv, a[3] * inv);
    *(u32x2*)(p.out + row * kHeadDim + 4 * dq) = w;
    if (p.lse && dq == 0) p.lse[row] = (m + fast_log2(l)) * kLn2;
  };
  // entry `index` of a table of partials with `pitch` entries per (sequence, head) row
  auto store_partial = [&](float* acc_tab, float* ml_tab, uint32_t pitch, uint32_t index, uint32_t h,
                           uint32_t dq, const f32x4& a, float l, float m) {
    const size_t prow = ((size_t)seq * p.n_q_heads + head0 + h) * pitch + index;
    store_coherent64(acc_tab + prow * kHeadDim + 4 * dq, a[0], a[1]);
    store_coherent64(acc_tab + prow * kHeadDim + 4 * dq + 2, a[2], a[3]);
    if (dq == 0) store_coherent64(ml_tab + prow * 2, m, l);
  };
#pragma unroll
  for (int n = 0; n < kItems; ++n) {
    const uint32_t item = tid + n * kThreads;
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
    if (p.n_split == 1)
      emit_final(h, dq, a, lsum, mmax);
    else
      store_partial(p.ws_acc, p.ws_ml, p.n_split, split, h, dq, a, lsum, mmax);
  }
  if (p.n_split == 1) return;

  // ---- the last workgroup to arrive merges: two levels, 16 partials each -----
  // Partials are written and read with agent-scope atomic accesses, which go
  // through to the device-wide point of coherence on their own (each XCD has
  // its own L2), so no cache write-back or invalidate is needed: a device-scope
  // fence costs a whole-L2 operation per wave and, with a thousand workgroups,
  // several times the kernel itself.  Ordering is explicit instead: every thread
  // waits until its own partial stores have been acknowledged, the workgroup
  // barrier collects all of them, and only then is the arrival counted; the
  // merging workgroup issues its loads only after the counter's return value
  // has been seen by all of its threads.
  // (Measured and dropped: tickets taken at the end of the key loop, the holder of the
  // last one keeping its partial in registers and waiting for a count of stored partials.
  // The ticket order is not the order of finishing, so the folder mostly waits for a
  // slower workgroup's store, count and its own poll: 0.3 us slower with one fold level,
  // 2.7 us with two.)
  // Splits are grouped in clusters of 16.  The last arrival of a cluster folds
  // its partials into one cluster partial; the last cluster to finish folds the
  // cluster partials into the output.  A merge is one workgroup reading from
  // L2/HBM, so its cost grows with the bytes it reads: two short levels keep
  // the tail of the launch at a few microseconds even with 256 splits a plane.
  const uint32_t live = min(p.n_split, (pos + p.split_len) / p.split_len);
  const uint32_t n_clusters = (live + kMergeFan - 1) / kMergeFan;
  const uint32_t cluster = split / kMergeFan;
  const uint32_t in_cluster = min((uint32_t)kMergeFan, live - cluster * kMergeFan);
  uint32_t* ctr = p.counters + ((size_t)seq * gridDim.y + blockIdx.y) * p.counters_per_plane;
  __shared__ uint32_t s_last;
  auto arrive = [&](uint32_t* c, uint32_t expected) -> bool {
    wait_vm_done();
    __syncthreads();
    if (tid == 0) {
      const uint32_t old = __hip_atomic_fetch_add(c, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      const uint32_t last = (old + 1 == expected) ? 1u : 0u;
      // back to zero for the next launch; nobody else touches it in this one
      if (last) __hip_atomic_store(c, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      s_last = last;
    }
    __syncthreads();
    return s_last != 0;
  };
  // Fold `count` (<= 16) partials of every head of this group, starting at partial `first`
  // of a table with `pitch` partials per row.  A thread issues every load its item needs
  // before it uses any: a fold costs one trip to memory, an 8-byte (max, sum) pair per
  // thread, shared through LDS, and one 16-byte accumulator quad per partial; the pairs come
  // back from LDS into registers in one go as well (read one by one inside the loops below,
  // every LDS round trip showed: 1.1 us for eight partials).
  // emit(h, dq, a[4], sum, max) receives columns 4 dq .. 4 dq + 3.
  auto fold = [&](const float* acc_tab, const float* ml_tab, uint32_t pitch, uint32_t first,
                  uint32_t count, auto emit) {
    float* sm = (float*)smem;  // [head][kMergeFan][2]; the reduction buffer is idle by now
    const __amdgpu_buffer_rsrc_t acc_rsrc = table_rsrc(acc_tab);
    const uint32_t n_ml = heads_here * count;
    const uint32_t h_e = tid / count, s_e = tid % count;
    uint64_t ml_bits = 0;
    if ((uint32_t)tid < n_ml)
      ml_bits = load_coherent64(
          ml_tab + (((size_t)seq * p.n_q_heads + head0 + h_e) * pitch + first + s_e) * 2);
#pragma unroll
    for (int n = 0; n < kItems; ++n) {
      const uint32_t item = tid + n * kThreads;
      const bool mine = item < n_items;
      const uint32_t h = mine ? item / kQuads : 0, dq = item % kQuads;
      // byte offset of entry `first`, columns 4 dq.. of this head's row (tables stay far below 4 GB)
      const uint32_t at =
          (uint32_t)(((((size_t)seq * p.n_q_heads + head0 + h) * pitch + first) * kHeadDim + 4 * dq) * 4);
      f32x4 av[kMergeFan];
#pragma unroll
      for (int i = 0; i < kMergeFan; ++i) {
        av[i] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
        if (mine && (uint32_t)i < count) av[i] = load_coherent128(acc_rsrc, at + (uint32_t)i * (kHeadDim * 4));
      }
      if (n == 0) {  // (every thread passes here once: the branch holds a barrier)
        if ((uint32_t)tid < n_ml) *(uint64_t*)(sm + (h_e * kMergeFan + s_e) * 2) = ml_bits;
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
  };

  if (!arrive(ctr + 1 + cluster, in_cluster)) return;
  if (n_clusters == 1) {
    fold(p.ws_acc, p.ws_ml, p.n_split, 0, live, emit_final);
    return;
  }
  fold(p.ws_acc, p.ws_ml, p.n_split, cluster * kMergeFan, in_cluster,
       [&](uint32_t h, uint32_t dq, const f32x4& a, float l, float m) {
         store_partial(p.ws2_acc, p.ws2_ml, p.n_cluster_max, cluster, h, dq, a, l, m);
       });
  if (!arrive(ctr, n_clusters)) return;
  fold(p.ws2_acc, p.ws2_ml, p.n_cluster_max, 0, n_clusters, emit_final);
}

}  // namespace

DecodePlan decode_plan(uint32_t max_len, uint32_t batch, uint32_t n_kv_heads, uint32_t n_cu) {
  // Two workgroups per compute unit measured best on MI355X (each workgroup has
  // fixed costs — query load, wave merge, partial write, arrival — that more,
  // shorter workgroups pay more often); never make a split shorter than four
  // 64-key steps.
  constexpr uint32_t per_cu = 2;
  const uint32_t target = n_cu * per_cu;
  const uint32_t planes = batch * n_kv_heads;
  // rounded down: a few workgroups beyond two per compute unit make some units host three, and
  // those finish half as late again (20 sequences x 8192: 67 us with 560 workgroups, 57 us with 480)
  const uint32_t want = target / planes > 0 ? target / planes : 1;
  uint32_t split_len = (max_len + want - 1) / want;
  split_len = (split_len + kDecodeStepKeys - 1) / kDecodeStepKeys * kDecodeStepKeys;
  if (split_len < 4 * kDecodeStepKeys) split_len = 4 * kDecodeStepKeys;
  // both merge levels fold at most 16 partials: at most 16 * 16 splits per plane
  const uint32_t floor_len =
      ((max_len + kMergeFan * kMergeFan - 1) / (kMergeFan * kMergeFan) + kDecodeStepKeys - 1) /
      kDecodeStepKeys * kDecodeStepKeys;
  if (split_len < floor_len) split_len = floor_len;
  DecodePlan plan;
  plan.split_len = split_len;
  plan.n_split = (max_len + split_len - 1) / split_len;
  return plan;
}

DecodeWorkspace decode_workspace(uint32_t batch_capacity, uint32_t n_q_heads, uint32_t n_kv_heads,
                                 uint32_t n_cu) {
  // rows = batch * heads * n_split with n_split <= ceil(4*n_cu / (batch*kv_heads))
  const size_t group = n_q_heads / n_kv_heads;
  DecodeWorkspace w;
  w.rows = (size_t)batch_capacity * n_q_heads + (size_t)n_cu * 16 * group;
  // cluster partials: ceil(n_split / 16) per row of batch * heads
  w.rows2 = w.rows / kMergeFan + (size_t)batch_capacity * n_q_heads;
  // counters: (1 + clusters) per plane, planes <= batch * heads
  w.counters = w.rows2 + (size_t)batch_capacity * n_q_heads;
  return w;
}

bool decode_plan_fits(const DecodeWorkspace& w, uint32_t batch, uint32_t n_q_heads,
                      uint32_t n_kv_heads, uint32_t group, uint32_t n_split) {
  const size_t n_cluster = (n_split + kMergeFan - 1) / kMergeFan;
  const size_t head_groups = (group + kMaxHeadsPerGroup - 1) / kMaxHeadsPerGroup;
  return (size_t)batch * n_q_heads * n_split <= w.rows &&
         (size_t)batch * n_q_heads * n_cluster <= w.rows2 &&
         (size_t)batch * n_kv_heads * head_groups * (1 + n_cluster) <= w.counters;
}

hipError_t launch_decode(const AttnArgs& a, hipStream_t stream) {
  DecodeKernelArgs p;
  p.q = (const uint16_t*)a.q;
  p.k = (const uint16_t*)a.k;
  p.v = (const uint16_t*)a.v;
  p.out = (uint16_t*)a.out;
  p.lse = a.lse;
  p.positions = a.positions;
  p.seq_offsets = a.seq_offsets;
  p.seq_caps = a.seq_caps;
  p.ws_acc = a.ws_acc;
  p.ws_ml = a.ws_ml;
  p.ws2_acc = a.ws2_acc;
  p.ws2_ml = a.ws2_ml;
  p.counters = a.counters;
  p.n_cluster_max = (a.n_split + kMergeFan - 1) / kMergeFan;
  p.counters_per_plane = 1 + p.n_cluster_max;
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
    hipLaunchKernelGGL((decode_split_kernel<F16>), grid, block, 0, stream, p);
  else
    hipLaunchKernelGGL((decode_split_kernel<BF16>), grid, block, 0, stream, p);
  return hipGetLastError();
}

}  // namespace ellm
