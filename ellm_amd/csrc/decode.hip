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

#include "decode_common.hpp"

namespace ellm {
using namespace dec;
namespace {

// PENDING = kPendSums: the launch of a fused step (ellm_matmul3_attn_run): the query rows and the
// new key / value row of every plane come as the projection's raw sums (p.pend) and are finished
// here.  kPendRows (ellm_kv_append_attn_run): the new key / value rows come as stored 16-bit rows.
template <typename T, int PENDING>
__global__ __launch_bounds__(kDecThreads, PENDING ? 2 : 4) void decode_split_kernel(DecodeKernelArgs p) {
  __shared__ __attribute__((aligned(16))) uint16_t smem[kDecWaves * kWaveLdsHalves];
  __shared__ uint32_t s_last;

  // The split a workgroup takes is rotated by its plane's number.  Workgroups are dealt to the
  // eight XCDs by their linear id; with the unrotated mapping (and a split count that is a
  // multiple of 8) one XCD would read the same stretch of every plane, and XCDs differ in how
  // fast they reach a given stretch of memory: 4 sequences x 32768 keys took 51.4 us
  // unrotated, 48.0 us rotated (16 x 8192: no difference).
  const uint32_t split = (blockIdx.x + blockIdx.y + gridDim.y * blockIdx.z) % gridDim.x;
  const uint32_t kvh = blockIdx.y / p.head_groups;
  const uint32_t hgrp = blockIdx.y % p.head_groups;
  const uint32_t seq = blockIdx.z;
  const Lane t;

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
  const uint32_t head0 = kvh * p.group + hgrp * kMaxHeadsPerGroup;
  const uint32_t row0 = seq * p.n_q_heads + head0;  // output row of the group's first head
  u32x4 qreg[4];
  float m_run, l_run;
  f32x4 acc[8];
  if constexpr (PENDING) {
    PendingQueries queries;   // requested first: the stream's own loads follow
    if constexpr (PENDING == kPendSums) queries.fetch(p.pend, seq, head0, pos, t, heads_here);
    // the split that holds the plane's last key takes the new row; one workgroup of a group writes it
    const NewRow fresh = new_row_of<PENDING>(p.pend, seq, kvh, pos, p.n_q_heads, p.n_kv_heads,
                                             const_cast<uint16_t*>(p.k) + plane + (size_t)pos * p.kv_stride_pos,
                                             const_cast<uint16_t*>(p.v) + plane + (size_t)pos * p.kv_stride_pos,
                                             k_end == len, hgrp == 0);
    if constexpr (PENDING == kPendRows) load_queries(p.q + (size_t)row0 * kHeadDim, t, heads_here, qreg);
    stream_keys<T, PENDING>(p.k + plane, p.v + plane, p.kv_stride_pos, k_begin, k_end, pos, qreg, smem, t,
                            split * 7u + blockIdx.y * 3u + seq * 5u, p.scale_log2, m_run, l_run, acc, &fresh,
                            PENDING == kPendSums ? &queries : nullptr, heads_here);
    // the finished query rows, once per group: by the workgroup that also wrote the new key
    if constexpr (PENDING == kPendSums) {
      if (fresh.present) store_queries(const_cast<uint16_t*>(p.q) + (size_t)row0 * kHeadDim, t, heads_here, qreg);
    }
  } else {
    load_queries(p.q + (size_t)row0 * kHeadDim, t, heads_here, qreg);
    stream_keys<T>(p.k + plane, p.v + plane, p.kv_stride_pos, k_begin, k_end, pos, qreg, smem, t,
                   split * 7u + blockIdx.y * 3u + seq * 5u, p.scale_log2, m_run, l_run, acc);
  }

  auto final_row = [&](uint32_t h, uint32_t dq, const f32x4& a, float l, float m) {
    emit_final<T>(p.out, p.lse, row0 + h, dq, a, l, m);
  };
  merge_waves(smem, t, heads_here, m_run, l_run, acc,
              [&](uint32_t h, uint32_t dq, const f32x4& a, float l, float m) {
                if (p.n_split == 1)
                  final_row(h, dq, a, l, m);
                else
                  store_partial(p.ws_acc, p.ws_ml, (size_t)((row0 + h) * p.n_split + split), dq, a, l, m);
              });
  if (p.n_split == 1) return;

  // ---- the last workgroup to arrive merges: two levels, 16 partials each -----
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

  if (!arrive(ctr + 1 + cluster, in_cluster, &s_last, t.tid)) return;
  if (n_clusters == 1) {
    fold(smem, t, heads_here, p.ws_acc, p.ws_ml, row0 * p.n_split, p.n_split, 1, live, final_row);
    return;
  }
  fold(smem, t, heads_here, p.ws_acc, p.ws_ml, row0 * p.n_split + cluster * kMergeFan, p.n_split, 1, in_cluster,
       [&](uint32_t h, uint32_t dq, const f32x4& a, float l, float m) {
         store_partial(p.ws2_acc, p.ws2_ml, (size_t)((row0 + h) * p.n_cluster_max + cluster), dq, a, l, m);
       });
  if (!arrive(ctr, n_clusters, &s_last, t.tid)) return;
  fold(smem, t, heads_here, p.ws2_acc, p.ws2_ml, row0 * p.n_cluster_max, p.n_cluster_max, 1, n_clusters,
       final_row);
}

}  // namespace

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
  p.batch = a.batch;
  p.scale_log2 = a.scale * kLog2e;
  p.pend = a.pending;

  dim3 grid(a.n_split, a.n_kv_heads * p.head_groups, a.batch);
  dim3 block(kDecThreads);
  if (a.pending.raw) {
    if (a.dtype == 0)
      hipLaunchKernelGGL((decode_split_kernel<F16, kPendSums>), grid, block, 0, stream, p);
    else
      hipLaunchKernelGGL((decode_split_kernel<BF16, kPendSums>), grid, block, 0, stream, p);
  } else if (a.pending.k_rows) {
    if (a.dtype == 0)
      hipLaunchKernelGGL((decode_split_kernel<F16, kPendRows>), grid, block, 0, stream, p);
    else
      hipLaunchKernelGGL((decode_split_kernel<BF16, kPendRows>), grid, block, 0, stream, p);
  } else if (a.dtype == 0) {
    hipLaunchKernelGGL((decode_split_kernel<F16, kPendNone>), grid, block, 0, stream, p);
  } else {
    hipLaunchKernelGGL((decode_split_kernel<BF16, kPendNone>), grid, block, 0, stream, p);
  }
  return hipGetLastError();
}

}  // namespace ellm
