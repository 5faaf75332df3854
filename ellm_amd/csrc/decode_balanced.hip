// Single-token attention for sequences of different lengths (ellm_attn_run_ragged: one
// position per sequence, read from device memory): the keys of all (sequence, kv head) planes,
// laid end to end, are dealt to the workgroups in equal shares.
//
// The kernel of decode.hip gives every plane the same number of splits of the same length,
// sized for the longest sequence the call may hold; with lengths spread between 1k and 128k
// (the single-token side of a mixed step) most workgroups then have a fraction of the longest
// one's keys or none at all.  Here the unit of work is 64 keys of one plane; plane p has
// u_p = ceil(length / 64) of them, all planes together U, and workgroup w of W takes units
// [w U / W, (w + 1) U / W) of the concatenation: a stretch of one plane, or the end of one plane,
// some whole planes and the start of another.  Each stretch (a "piece") runs the same stream, wave
// merge and, where a plane has more than one piece, the same partial / arrival / fold steps as
// the other kernel.  Everything a workgroup needs to know about the others (which workgroups share
// a plane, how many pieces it has, where their partials are) follows from the lengths alone, which
// every workgroup reads for itself: no queue, no claim counter, and the same split of the work,
// hence the same bits, whenever the lengths are the same.
//
// Reference semantics unchanged: per (sequence, query head) the result of flash_attention
// (src/kernel/x86_64/f16_512/flash_attention.rs:30-92) over keys 0..=position of the sequence.
#include "decode_common.hpp"
#include "decode_shares.hpp"

namespace ellm {
using namespace dec;
namespace {

constexpr uint32_t kUnitKeys = kDecodeStepKeys;   // 64: one step of the four waves
constexpr uint32_t kMaxBatch = 1024;              // lengths are scanned in LDS
static_assert(kBalancedFan == (uint32_t)kMergeFan, "decode_shares.hpp numbers the slots for this fan");

// (the compiler cannot see that a value every lane computes alike is wave-uniform)
__device__ __forceinline__ uint32_t uni(uint32_t v) { return (uint32_t)__builtin_amdgcn_readfirstlane((int)v); }

// Pieces of plane p occupy consecutive partial slots first_w(p) + p .. (the pair (workgroup,
// plane) moves on by one in exactly one of the two from piece to piece, so workgroup + plane
// numbers the pieces of a launch without gaps that matter and without collisions); a plane's
// clusters of 16 pieces take cluster slots p + slot0 / 16 + c, which are distinct for the same
// reason (1 + floor(n / 16) >= ceil(n / 16)).

// PENDING: the launch of a fused step, as in decode.hip.
template <typename T, int PENDING>
__global__ __launch_bounds__(kDecThreads, 2) void decode_balanced_kernel(DecodeKernelArgs p) {
  __shared__ __attribute__((aligned(16))) uint16_t smem[kDecWaves * kWaveLdsHalves];
  __shared__ uint32_t prefix[kMaxBatch + 1];   // units of the sequences before sequence b (per plane)
  __shared__ uint32_t s_pos[kMaxBatch];        // last position of every sequence
  __shared__ uint32_t s_last, s_umax, s_umin;
  const Lane t;
  const uint32_t B = p.batch;

  auto position_of = [&](uint32_t b) {
    uint32_t pos = min(p.positions[b], p.position);
    if (p.seq_caps) pos = min(pos, p.seq_caps[b] - 1);
    return pos;
  };
  // Units per sequence and their running sum.  Up to 64 sequences: every wave keeps them in
  // registers, sequence b in lane b (no LDS, no barrier, and the look-up below is a ballot);
  // more: wave 0 scans them into LDS, 64 at a time.
  auto wave_scan = [&](uint32_t v) {   // inclusive sum over the lanes below and this one
#pragma unroll
    for (int d = 1; d < kWave; d <<= 1) {
      const uint32_t below = __shfl_up(v, d, kWave);
      if (t.lane >= d) v += below;
    }
    return v;
  };
  auto wave_max = [&](uint32_t v) {
#pragma unroll
    for (int d = 1; d < kWave; d <<= 1) v = max(v, (uint32_t)__shfl_xor(v, d, kWave));
    return v;
  };
  auto wave_min = [&](uint32_t v) {
#pragma unroll
    for (int d = 1; d < kWave; d <<= 1) v = min(v, (uint32_t)__shfl_xor(v, d, kWave));
    return v;
  };
  auto lane_value = [&](uint32_t v, uint32_t l) { return (uint32_t)__builtin_amdgcn_readlane((int)v, (int)l); };
  const bool in_registers = B <= (uint32_t)kWave;   // (uniform)
  uint32_t r_pos = 0, r_units = 0, r_incl = 0, total_units, umax_all, umin_all;
  if (in_registers) {
    const bool live = (uint32_t)t.lane < B;
    r_pos = live ? position_of(t.lane) : 0u;
    r_units = live ? r_pos / kUnitKeys + 1 : 0u;
    r_incl = wave_scan(r_units);
    total_units = lane_value(r_incl, kWave - 1);
    umax_all = uni(wave_max(r_units));
    umin_all = uni(wave_min(live ? r_units : 0xffffffffu));
  } else {
    if (t.wave == 0) {
      uint32_t carry = 0, umax = 0, umin = 0xffffffffu;
      for (uint32_t base = 0; base < B; base += kWave) {
        const bool live = base + t.lane < B;
        const uint32_t pos_b = live ? position_of(base + t.lane) : 0u;
        if (live) s_pos[base + t.lane] = pos_b;
        const uint32_t u = live ? pos_b / kUnitKeys + 1 : 0u;
        const uint32_t incl = wave_scan(u);
        if (live) prefix[base + t.lane + 1] = carry + incl;
        carry += __shfl(incl, kWave - 1, kWave);
        umax = max(umax, wave_max(u));
        umin = min(umin, wave_min(live ? u : 0xffffffffu));
      }
      if (t.lane == 0) {
        prefix[0] = 0;
        s_umax = umax;
        s_umin = umin;
      }
    }
    __syncthreads();
    total_units = uni(prefix[B]);
    umax_all = uni(s_umax);
    umin_all = uni(s_umin);
  }

  // All of the index arithmetic is 32-bit (the launcher keeps calls with 2^31 units or more
  // away): a 64-bit division is a subroutine of a few hundred instructions, and a handful of
  // them per piece showed as 2 us on a 47 us launch.
  const uint32_t PL = p.n_kv_heads * p.head_groups;   // planes per sequence
  const uint32_t U = PL * total_units;
  // workgroups that take part: at most one per unit, and few enough that no plane is cut
  // into more pieces than two fold levels take.
  // Planes of equal length (to the unit): a whole number of workgroups per plane, so that the
  // shares below end where the planes end and no workgroup starts a second piece (24 sequences
  // x 8192 keys: 96 planes, 480 workgroups of 5 pieces a plane instead of 512 shares of 5.33).
  // Else a multiple of eight, for the XCD order below.
  // One workgroup per compute unit streams as fast as two that share one, leaves half the
  // partial rows to fold and ends more evenly (32 sequences of 1k-128k keys: 658 against 679 us);
  // two per unit are better where the rounding above would leave units idle (96 equal planes:
  // 192 of 256) and where a workgroup walks several short planes one after the other, each with
  // its own start-up that a second workgroup on the unit hides (400 planes of 100-4096 keys).
  // (decode_shares.hpp: balanced_workgroups, also walked by the CPU tests)
  const uint32_t planes_all = PL * B;
  const uint32_t W = balanced_workgroups(gridDim.x, p.wgs_one, U, umax_all, umin_all, planes_all);
  // Workgroups are dealt to the eight XCDs by their id modulo 8.  Each XCD takes one contiguous
  // eighth of the shares, so that no two of them walk the same stretch of memory side by side
  // (with shares numbered like the workgroups and as many pieces per plane as XCDs, every XCD
  // would read the same stretch of every plane).
  if (blockIdx.x >= W) return;
  const uint32_t w = balanced_share_of(blockIdx.x, W);
  // share g begins at floor(g U / W) (decode_shares.hpp): equal to the unit, and for equal planes
  // with W a multiple of their number a plane's end is a share's end
  const Shares shares(W, U);
  auto share_begin = [&](uint32_t g) { return shares.begin(g); };
  auto holder = [&](uint32_t unit) { return shares.holder(unit); };
  const uint32_t G = min((uint32_t)kMaxHeadsPerGroup, p.group);   // partial rows per slot
  // cluster partials and their counters are indexed by cluster slot; the planes' own counters
  // follow the cluster counters
  uint32_t* const plane_ctrs = p.counters + p.n_cluster_max;

  uint32_t x = share_begin(w);
  const uint32_t x_end = share_begin(w + 1);
  while (x < x_end) {
    // the sequence that holds unit x: the last b with PL prefix[b] <= x
    // (every thread computes the same values; readfirstlane tells the compiler so)
    uint32_t seq, u_seq, seq_start, pos;
    if (in_registers) {
      const uint64_t ended = __ballot((uint32_t)t.lane < B && PL * r_incl <= x);   // sequences that end at or before x
      seq = (uint32_t)__builtin_popcountll(ended);
      u_seq = lane_value(r_units, seq);
      seq_start = PL * (lane_value(r_incl, seq) - u_seq);
      pos = lane_value(r_pos, seq);
    } else {
      uint32_t lo = 0, hi = B;
      while (hi - lo > 1) {
        const uint32_t mid = (lo + hi) >> 1;
        if (PL * prefix[mid] <= x)
          lo = mid;
        else
          hi = mid;
      }
      seq = uni(lo);
      u_seq = uni(prefix[seq + 1] - prefix[seq]);
      seq_start = uni(PL * prefix[seq]);
      pos = uni(s_pos[seq]);
    }
    const uint32_t r = x - seq_start;
    const uint32_t pl = r / u_seq, a = r - pl * u_seq;        // plane of the sequence, first unit in it
    const uint32_t S = seq_start + pl * u_seq, E = S + u_seq;
    const uint32_t stop = min(x_end, E);
    const uint32_t a_end = a + (stop - x);
    // the workgroups that hold the plane's first and last unit (this one, when the piece starts
    // or ends with the plane: no look-up then)
    const uint32_t first_w = x == S ? w : holder(S);
    const uint32_t last_w = stop == E ? w : holder(E - 1);
    const uint32_t n_pieces = last_w - first_w + 1, piece = w - first_w;
    const uint32_t plane_id = seq * PL + pl;
    const uint32_t slot0 = balanced_slot0(first_w, plane_id);

    const uint32_t k_begin = a * kUnitKeys;
    const uint32_t k_end = min(pos + 1, a_end * kUnitKeys);
    const uint32_t kvh = pl / p.head_groups, hgrp = pl % p.head_groups;
    const uint32_t heads_here = min((uint32_t)kMaxHeadsPerGroup, p.group - hgrp * kMaxHeadsPerGroup);
    const size_t plane = seq_plane_offset(p.seq_offsets, p.kv_stride_seq, seq) + kvh * p.kv_stride_head;
    const uint32_t head0 = kvh * p.group + hgrp * kMaxHeadsPerGroup;
    const uint32_t row0 = seq * p.n_q_heads + head0;
    u32x4 qreg[4];
    float m_run, l_run;
    f32x4 acc[8];
    if constexpr (PENDING) {
      PendingQueries queries;   // requested first: the stream's own loads follow
      if constexpr (PENDING == kPendSums) queries.fetch(p.pend, seq, head0, pos, t, heads_here);
      // the piece that holds the plane's last key takes the new row; one workgroup of a group writes it
      const NewRow fresh = new_row_of<PENDING>(p.pend, seq, kvh, pos, p.n_q_heads, p.n_kv_heads,
                                               const_cast<uint16_t*>(p.k) + plane + (size_t)pos * p.kv_stride_pos,
                                               const_cast<uint16_t*>(p.v) + plane + (size_t)pos * p.kv_stride_pos,
                                               k_end == pos + 1, hgrp == 0);
      if constexpr (PENDING == kPendRows) load_queries(p.q + (size_t)row0 * kHeadDim, t, heads_here, qreg);
      stream_keys<T, PENDING>(p.k + plane, p.v + plane, p.kv_stride_pos, k_begin, k_end, pos, qreg, smem, t,
                              w * 7u + pl * 3u + seq * 5u, p.scale_log2, m_run, l_run, acc, &fresh,
                              PENDING == kPendSums ? &queries : nullptr, heads_here);
      if constexpr (PENDING == kPendSums) {
        if (fresh.present) store_queries(const_cast<uint16_t*>(p.q) + (size_t)row0 * kHeadDim, t, heads_here, qreg);
      }
    } else {
      load_queries(p.q + (size_t)row0 * kHeadDim, t, heads_here, qreg);
      stream_keys<T>(p.k + plane, p.v + plane, p.kv_stride_pos, k_begin, k_end, pos, qreg, smem, t,
                     w * 7u + pl * 3u + seq * 5u, p.scale_log2, m_run, l_run, acc);
    }

    auto final_row = [&](uint32_t h, uint32_t dq, const f32x4& av, float l, float m) {
      emit_final<T>(p.out, p.lse, (size_t)(row0 + h), dq, av, l, m);
    };
    merge_waves(smem, t, heads_here, m_run, l_run, acc,
                [&](uint32_t h, uint32_t dq, const f32x4& av, float l, float m) {
                  if (n_pieces == 1)
                    final_row(h, dq, av, l, m);
                  else
                    store_partial(p.ws_acc, p.ws_ml, (size_t)((slot0 + piece) * G + h), dq, av, l, m);
                });
    if (n_pieces > 1) {
      const uint32_t n_clusters = (n_pieces + kMergeFan - 1) / kMergeFan;
      const uint32_t cluster = piece / kMergeFan;
      const uint32_t in_cluster = min((uint32_t)kMergeFan, n_pieces - cluster * kMergeFan);
      const uint32_t cslot0 = balanced_cluster_slot0(slot0, plane_id);
      if (arrive(p.counters + cslot0 + cluster, in_cluster, &s_last, t.tid)) {
        if (n_clusters == 1) {
          fold(smem, t, heads_here, p.ws_acc, p.ws_ml, slot0 * G, 1, G, n_pieces, final_row);
        } else {
          fold(smem, t, heads_here, p.ws_acc, p.ws_ml, (slot0 + cluster * kMergeFan) * G, 1, G, in_cluster,
               [&](uint32_t h, uint32_t dq, const f32x4& av, float l, float m) {
                 store_partial(p.ws2_acc, p.ws2_ml, (size_t)((cslot0 + cluster) * G + h), dq, av, l, m);
               });
          if (arrive(plane_ctrs + plane_id, n_clusters, &s_last, t.tid))
            fold(smem, t, heads_here, p.ws2_acc, p.ws2_ml, cslot0 * G, 1, G, n_clusters, final_row);
        }
      }
    }
    x = uni(stop);
    __syncthreads();   // the next piece writes the staging buffers that the merge steps read
  }
}

}  // namespace

// Whether a call with per-sequence positions goes to the balanced kernel: enough keys that the
// split matters (below, the other kernel's fixed plan costs nothing and starts sooner), a batch
// whose lengths fit the scan, and a workspace that holds the partials, cluster partials and
// counters of `wgs` workgroups.
bool decode_balanced_takes(const DecodeWorkspace& w, uint32_t batch, uint32_t n_kv_heads, uint32_t group,
                           uint32_t max_len, uint32_t wgs) {
  if (batch > kMaxBatch) return false;
  const uint64_t head_groups = (group + kMaxHeadsPerGroup - 1) / kMaxHeadsPerGroup;
  const uint64_t planes = (uint64_t)batch * n_kv_heads * head_groups;
  const uint64_t units = planes * ((max_len + kUnitKeys - 1) / kUnitKeys);
  if (units < 8ull * wgs || units + wgs >= (1ull << 31) || wgs >= (1u << 16)) return false;
  const uint64_t G = group < (uint32_t)kMaxHeadsPerGroup ? group : (uint32_t)kMaxHeadsPerGroup;
  const uint64_t slots = balanced_slots(wgs, (uint32_t)planes), cslots = balanced_cluster_slots(wgs, (uint32_t)planes);
  return slots * G <= w.rows && cslots * G <= w.rows2 && cslots + planes <= w.counters;
}

hipError_t launch_decode_balanced(const AttnArgs& a, uint32_t wgs, hipStream_t stream) {
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
  p.kv_stride_seq = a.kv_stride_seq;
  p.kv_stride_head = a.kv_stride_head;
  p.kv_stride_pos = a.kv_stride_pos;
  p.n_q_heads = a.n_q_heads;
  p.n_kv_heads = a.n_kv_heads;
  p.group = a.group;
  p.head_groups = (a.group + kMaxHeadsPerGroup - 1) / kMaxHeadsPerGroup;
  p.position = a.position_index;
  p.split_len = 0;
  p.n_split = 0;
  p.batch = a.batch;
  p.wgs_one = a.n_cu ? a.n_cu : wgs;
  p.scale_log2 = a.scale * kLog2e;
  // cluster slots (the kernel's cslot0 + cluster stays below this): the planes' own counters follow
  const uint32_t planes = a.batch * a.n_kv_heads * p.head_groups;
  p.n_cluster_max = balanced_cluster_slots(wgs, planes);
  p.counters_per_plane = 0;
  p.pend = a.pending;
  const dim3 grid(wgs), block(kDecThreads);
  if (a.pending.raw) {
    if (a.dtype == 0)
      hipLaunchKernelGGL((decode_balanced_kernel<F16, kPendSums>), grid, block, 0, stream, p);
    else
      hipLaunchKernelGGL((decode_balanced_kernel<BF16, kPendSums>), grid, block, 0, stream, p);
  } else if (a.pending.k_rows) {
    if (a.dtype == 0)
      hipLaunchKernelGGL((decode_balanced_kernel<F16, kPendRows>), grid, block, 0, stream, p);
    else
      hipLaunchKernelGGL((decode_balanced_kernel<BF16, kPendRows>), grid, block, 0, stream, p);
  } else if (a.dtype == 0) {
    hipLaunchKernelGGL((decode_balanced_kernel<F16, kPendNone>), grid, block, 0, stream, p);
  } else {
    hipLaunchKernelGGL((decode_balanced_kernel<BF16, kPendNone>), grid, block, 0, stream, p);
  }
  return hipGetLastError();
}

}  // namespace ellm
