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
//   O^T[d][row]  += V^T . P^T   32x32x16 MFMA, A = V^T from LDS (transposing read), B = P^T in registers
// The C layout of S^T (lane = row, registers = keys) is, up to a fixed
// permutation of keys inside each 16-key group, the B layout the second MFMA
// wants; the V^T operand is read with the same permutation, so P never leaves the
// lane that produced it and row max / row sum need one cross-lane exchange.
//
// A workgroup (8 waves) owns 8 blocks of 32 query rows that all read the same
// K/V plane: up to 8 query heads of one GQA group x consecutive token blocks.
// Stacking the group's heads makes each LDS tile feed 8 times more MFMA work
// and keeps the token span (and so the masked part of the diagonal tile) short.
#include <type_traits>

#include "chunk_plan.hpp"
#include "common.hpp"
#include "kernels.hpp"

namespace ellm {
namespace {

constexpr int kBK = 64;                     // keys per tile
constexpr int kKsPitch = kHeadDim + 8;      // halves per K row (272 B)
constexpr int kKsHalves = kBK * kKsPitch;
constexpr float kRescaleStep = 8.0f;        // log2 units

struct PrefillKernelArgs {
  const uint16_t* q;
  const uint16_t* k;
  const uint16_t* v;
  uint16_t* out;
  float* lse;
  size_t q_token_stride;  // elements between consecutive tokens of Q/O
  size_t kv_stride_seq, kv_stride_head, kv_stride_pos;
  const size_t* seq_offsets;  // per-sequence plane offsets (null: sequence x kv_stride_seq)
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
  // Key range split over gridDim.y workgroups (few row blocks on a long cache): split s
  // walks tiles [s * split_tiles, (s + 1) * split_tiles) and leaves, per query row, its
  // unnormalised output row, running maximum (log2 units) and denominator in
  // part_o [row][n_split][128] / part_ml [row][n_split][2] for prefill_merge_kernel.
  uint32_t n_split, split_tiles;
  float* part_o;
  float* part_ml;
};

// ---------------------------------------------------------------------------
// Ping-pong kernel: 8 waves, two per SIMD.  Waves 0-3 and waves 4-7 run the
// same per-tile sequence  S^T = K.Q^T -> soft-max -> O^T += V^T.P^T  half a
// step apart: while one group is in its matrix phase (P.V of the previous tile,
// then Q.K of the next one, plus moving the following K or V tile into LDS) the
// other group is in its vector phase (mask, row max, exponentials, packing), and
// a workgroup barrier flips the roles.  Two waves that share a SIMD are thus
// never both in the same phase, which is what lets the MFMA pipe and the vector
// ALU work at the same time; left to themselves, two identical workgroups on a
// compute unit run in lockstep and the two pipes take turns instead.
// Rows: wave w owns row block w (32 rows) of 8; all 256 rows read the same K/V
// tiles.  Waves 0-3 stage the K tiles, waves 4-7 the V tiles.
// ---------------------------------------------------------------------------
__device__ __forceinline__ uint64_t uniform64(const void* p) {  // the compiler cannot see that p is wave-uniform
  const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(uint64_t)p);
  const uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)((uint64_t)p >> 32));
  return ((uint64_t)hi << 32) | (uint64_t)lo;
}
// Bytes a buffer descriptor may cover from byte `off` of a plane whose last visible byte ends at
// `valid`: what is left, capped at the 32 bits the descriptor's size field has (a tile or chunk
// reaches at most 64 rows beyond `off`, far less than that).  Both offsets are 64-bit: a plane
// of the reference's own [position][sequence][kv_head][128] state spans more than 2^32 bytes at
// 33 sequences x 131072 positions.  Scalar arithmetic (the arguments are wave-uniform).
__device__ __forceinline__ uint32_t bytes_left(uint64_t valid, uint64_t off) {
  const uint64_t left = valid > off ? valid - off : 0;
  const uint32_t capped = left > 0xffffffffull ? 0xffffffffu : (uint32_t)left;
  return (uint32_t)__builtin_amdgcn_readfirstlane((int)capped);
}
__device__ __forceinline__ uint64_t uniform_u64(uint64_t v) {
  const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)v);
  const uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(v >> 32));
  return ((uint64_t)hi << 32) | (uint64_t)lo;
}
typedef __attribute__((address_space(3))) uint16_t LdsHalf;
typedef __attribute__((address_space(3))) u32x4 LdsU32x4;
typedef __attribute__((address_space(3))) u32x2 LdsU32x2;
typedef short i16x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) i16x4 LdsI16x4;
// V rows in LDS: 288 B apart, so that the four rows a 16-lane block of a
// transposing read touches (32 B of each) fall into disjoint banks
constexpr int kVsPitch = kHeadDim + 16;
constexpr int kVsHalves = kBK * kVsPitch;
constexpr int kPpWaves = 8;
constexpr int kPpThreads = kPpWaves * kWave;
constexpr int kLdsAhead = 8;  // LDS operand reads in flight ahead of their MFMA
constexpr int kBufferFlags = 0x00020000;  // raw buffer of 32-bit data, no swizzle (word 3 of the descriptor)

template <typename T, bool SPLIT>
__global__ __launch_bounds__(kPpThreads, 2) void prefill_pingpong_kernel(PrefillKernelArgs p) {
  // K tiles [2][64][kKsPitch] then V tiles [3][64][kVsPitch]: V is staged one step
  // earlier than it is read, so that every operand of a matrix step is in LDS a whole
  // phase before the step starts and can be requested ahead of the barrier.
  __shared__ __attribute__((aligned(16))) uint16_t smem[2 * kKsHalves + 3 * kVsHalves];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = tid >> 6;
  const int j = lane & 31, g = lane >> 5;
  const int grp = wave >> 2;  // 0: waves 0-3, 1: waves 4-7

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
  const uint32_t kmax = P0 + wg_last_tok;
  const uint32_t all_tiles = kmax / kBK + 1;
  // the tiles of this workgroup: all of them, or its share of the key range
  const uint32_t kt0 = SPLIT ? blockIdx.y * p.split_tiles : 0u;
  if (SPLIT && kt0 >= all_tiles) return;  // (prefill_merge_kernel derives the live splits the same way)
  const uint32_t n_tiles = SPLIT ? min(all_tiles - kt0, p.split_tiles) : all_tiles;

  const uint32_t hg = wave % p.heads_per_wg, tb = wave / p.heads_per_wg;
  const uint32_t head = kvh * p.group + hgrp * p.heads_per_wg + hg;
  const uint32_t tok0 = t_base + 32 * tb;
  const uint32_t tok = min(tok0 + j, S - 1);
  const bool row_valid = tok0 + j < S;
  const uint32_t rowpos = P0 + tok;
  const uint32_t first_pos = P0 + min(tok0, S - 1);  // lowest position in this row block

  u32x4 qreg[8];
  {
    const uint16_t* qrow =
        p.q + (size_t)tok * p.q_token_stride + ((size_t)seq * p.n_q_heads + head) * kHeadDim;
#pragma unroll
    for (int s = 0; s < 8; ++s) {
      qreg[s] = load16(qrow + 16 * s + 8 * g);
      if (p.negate_q) qreg[s] ^= 0x80008000u;
    }
  }
  const float c = p.c;

  const size_t plane_at = seq_plane_offset(p.seq_offsets, p.kv_stride_seq, seq) + kvh * p.kv_stride_head;
  const uint16_t* kplane = p.k + plane_at;
  const uint16_t* vplane = p.v + plane_at;

  // staging: the 256 threads of a group move one 64 x 128 tile, four 16-byte pieces
  // each (rows ld_r + 16 i, columns 8 ld_c ..), K and V alike: V sits in LDS row by
  // row as it does in memory and is transposed by the LDS read (ds_read_b64_tr_b16).
  const int st_tid = tid & 255;
  const int ld_c = st_tid & 15, ld_r = st_tid >> 4;
  const uint16_t* plane = grp ? vplane : kplane;                  // wave-uniform
  const uint32_t stride_pos = (uint32_t)p.kv_stride_pos;
  // Tiles are fetched with buffer loads: the descriptor (base of tile kt, bytes
  // left up to the last key this workgroup may see) is scalar arithmetic, the
  // per-lane byte offsets of the four pieces never change, and rows past the
  // last key read as zero instead of needing a clamp: no vector instruction
  // per load.  The plane base goes through readfirstlane because the compiler
  // cannot see that it is wave-uniform.
  // (readfirstlane returns a signed int: the casts keep the low word from sign-extending)
  const uint32_t plane_lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(uint64_t)plane);
  const uint32_t plane_hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)((uint64_t)plane >> 32));
  const uint64_t plane_u = ((uint64_t)plane_hi << 32) | (uint64_t)plane_lo;
  const uint32_t tile_bytes = kBK * stride_pos * 2;   // (API bound: 64 rows span < 2^32 bytes)
  const uint64_t valid_bytes = uniform_u64(((uint64_t)kmax * stride_pos + kHeadDim) * 2);
  uint32_t piece_off[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) piece_off[i] = ((ld_r + 16 * i) * stride_pos + 8 * ld_c) * 2;
  // LDS addresses are kept as byte offsets: the buffers span more than the 64 KB an
  // instruction's immediate offset reaches, so each step forms one base register
  // per tile (step_base) and everything else is an immediate on top of it.
  const uint32_t lds0 = (uint32_t)(uintptr_t)(LdsHalf*)smem;
  auto step_base = [](uint32_t addr) {
    asm volatile("" : "+v"(addr));  // opaque: keeps the compiler from folding the sum another way
    return addr;
  };
  const uint32_t ks_store = lds0 + 2 * (ld_r * kKsPitch + 8 * ld_c);
  const uint32_t vs_store = lds0 + 2 * (2 * kKsHalves + ld_r * kVsPitch + 8 * ld_c);
  u32x4 stg[4];
  auto load_piece = [&](uint32_t kt, int i) {  // kt (relative to kt0) must be wave-uniform to the compiler
    const uint64_t off = (uint64_t)(kt0 + kt) * tile_bytes;
    const uint32_t left = bytes_left(valid_bytes, off);
    const __amdgpu_buffer_rsrc_t rsrc =
        __builtin_amdgcn_make_buffer_rsrc((void*)(plane_u + off), 0, left, kBufferFlags);
    stg[i] = __builtin_amdgcn_raw_buffer_load_b128(rsrc, piece_off[i], 0, 0);
  };
  // (the group comes as a compile-time constant where the caller runs behind the scalar
  // branch on the group, as the run-time value in the prologue)
  // base: step_base of this lane's place in the destination buffer
  auto store_piece = [&](auto group, uint32_t base, int i) {
    *(LdsU32x4*)(base + 2 * 16 * i * (group ? kVsPitch : kKsPitch)) = stg[i];
  };
  auto load_tile = [&](uint32_t kt) {
#pragma unroll
    for (int i = 0; i < 4; ++i) load_piece(kt, i);
  };
  auto store_base = [&](auto group, int buf) {
    return step_base(group ? vs_store + 2 * buf * kVsHalves : ks_store + 2 * buf * kKsHalves);
  };
  auto store_tile = [&](int buf) {
    const uint32_t base = store_base(grp, buf);
#pragma unroll
    for (int i = 0; i < 4; ++i) store_piece(grp, base, i);
  };

  float m_run = -INFINITY, l_run = 0.0f;
  f32x16 oacc[4];
#pragma unroll
  for (int db = 0; db < 4; ++db)
#pragma unroll
    for (int r = 0; r < 16; ++r) oacc[db][r] = 0.0f;
  f32x16 st[2];
  u32x4 pk[4];
#pragma unroll
  for (int cc = 0; cc < 4; ++cc) pk[cc] = u32x4{0u, 0u, 0u, 0u};  // P(-1) = 0

  // Every matrix step runs the same straight-line code, the first and the last
  // included: step 0 multiplies P(-1) = 0 by a zeroed "V(-1)" buffer, step n_tiles
  // multiplies Q by whatever finite K tile its buffer still holds and nobody reads
  // the result; tiles past the last one are fetched as zeros (the buffer
  // descriptor has no bytes left) and stored where nothing reads them.
  // prologue: K(0) and V(0) into LDS, K(1) and V(1) on their way into the staging
  // registers, zeros into the V^T buffer that step 0 reads.
  if (grp) {
#pragma unroll
    for (int i = 0; i < 4; ++i) stg[i] = u32x4{0u, 0u, 0u, 0u};
    store_tile(2);
  }
  load_tile(0);
  store_tile(0);
  load_tile(1);
  __syncthreads();

  // Matrix step kt = P.V of tile kt-1 and Q.K of tile kt, their MFMAs interleaved
  // (six accumulator chains instead of four or two, so no MFMA waits on the
  // one before it); then the group stores its tile kt+1 (group 0: K, group 1: V)
  // and fetches tile kt+2.  K(kt) sits in buffer kt % 2, V(kt) in buffer kt % 3: V is
  // staged one step before the first step that reads it, so that all operands of
  // a matrix step are in LDS a whole phase before it starts.  Operands come from
  // LDS kLdsAhead reads ahead of the MFMA that consumes them: issued just in
  // time, every pair of MFMAs (64 cycles) would wait out a full LDS round trip
  // (100+ cycles).  The first kLdsAhead are requested before the barrier that
  // opens the step (prefetch_ring), so the round trip overlaps the barrier wait.
  // A operand of P.V (rows = 32 dims, 16 keys): lane (dim j, key half g) holds keys
  // {4g..4g+3, 8+4g..8+4g+3} of the 16, the order in which the soft-max leaves P in
  // registers.  ds_read_b64_tr_b16 hands lane t of a 16-lane block element
  // (t & 3) of what lanes 4e + (t >> 2), e = 0..3, of that block address: with lane
  // s pointing at key s >> 2, dims 4 (s & 3).. of the block's 16 dims, lane t ends
  // up with dim t of 4 consecutive keys.  Two such reads (keys +0 and +8) make one operand.
  const uint32_t k_read = lds0 + 2 * (j * kKsPitch + 8 * g);
  const uint32_t v_read = lds0 + 2 * (2 * kKsHalves + (4 * g + ((lane & 15) >> 2)) * kVsPitch +
                                      16 * ((lane >> 4) & 1) + 4 * (lane & 3));
  auto mod3 = [](uint32_t x) { return x % 3u; };
  // operand n of the stream of matrix step kt: P.V 0, Q.K 0, P.V 1, Q.K 1, ...
  // (lane part of the address once per step, operand part as a compile-time offset)
  auto stream_operand = [&](uint32_t ks, uint32_t vs, int n) {
    const int i = n >> 1;
    if (n & 1) {  // K rows: i = 2 s + mb
      const int s = i >> 1, mb = i & 1;
      return (u32x4) * (const LdsU32x4*)(ks + 2 * (32 * mb * kKsPitch + 16 * s));
    }
    // V: i = 4 cc + db, keys 16 cc.., dims 32 db..
    const int cc = i >> 2, db = i & 3;
    const uint32_t at = vs + 2 * (16 * cc * kVsPitch + 32 * db);
    const i16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LdsI16x4*)at);
    const i16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LdsI16x4*)(at + 2 * 8 * kVsPitch));
    const u32x2 l2 = __builtin_bit_cast(u32x2, lo), h2 = __builtin_bit_cast(u32x2, hi);
    return u32x4{l2[0], l2[1], h2[0], h2[1]};
  };
  u32x4 ring[kLdsAhead];
  auto prefetch_ring = [&](uint32_t kt) __attribute__((always_inline)) {
    const uint32_t ks = step_base(k_read + 2 * (kt & 1) * kKsHalves);
    const uint32_t vs = step_base(v_read + 2 * mod3(kt + 2) * kVsHalves);  // V(kt-1)
#pragma unroll
    for (int n = 0; n < kLdsAhead; ++n) ring[n] = stream_operand(ks, vs, n);
  };
  auto matrix_step = [&](auto group, uint32_t kt) __attribute__((always_inline)) {
    const uint32_t ks = step_base(k_read + 2 * (kt & 1) * kKsHalves);
    const uint32_t vs = step_base(v_read + 2 * mod3(kt + 2) * kVsHalves);
    const uint32_t store_at = store_base(group, group ? (int)mod3(kt + 1) : (int)((kt + 1) & 1));
    // staging work is dealt out between the MFMAs, and a full scheduling barrier
    // after every MFMA keeps the compiler from regrouping any of it
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int n = 0; n < 32; ++n) {
      const int i = n >> 1;
      if (n & 1) {
        const int s = i >> 1, mb = i & 1;
        if (s == 0) {
          f32x16 z;
#pragma unroll
          for (int r = 0; r < 16; ++r) z[r] = 0.0f;
          st[mb] = Mfma<T>::m32x32x16(ring[n % kLdsAhead], qreg[s], z);
        } else {
          st[mb] = Mfma<T>::m32x32x16(ring[n % kLdsAhead], qreg[s], st[mb]);
        }
      } else {
        oacc[i & 3] = Mfma<T>::m32x32x16(ring[n % kLdsAhead], pk[i >> 2], oacc[i & 3]);
      }
      if (n + kLdsAhead < 32) ring[n % kLdsAhead] = stream_operand(ks, vs, n + kLdsAhead);
      // staging last: the loads issued at the end of the previous matrix step have had
      // almost a whole iteration (~2 us) to arrive before their registers are stored
      if (n >= 24 && n < 28) store_piece(group, store_at, n - 24);
      if (n >= 28 && n < 32) load_piece(kt + 2, n - 28);
      __builtin_amdgcn_sched_barrier(0);
    }
    // the barrier that follows carries no wait of its own: wait here for the LDS stores
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  };

  // Vector step kt = soft-max of tile kt: mask on the diagonal, row max, lazy
  // rescale of O^T, exponentials, packing, row sum.
  auto vector_step = [&](uint32_t kt) __attribute__((always_inline)) {
    const uint32_t kb = (kt0 + kt) * kBK;
    if (kb + kBK - 1 > first_pos) {  // tile crosses this row block's diagonal
#pragma unroll
      for (int mb = 0; mb < 2; ++mb)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const uint32_t key = kb + 32 * mb + 8 * (r >> 2) + 4 * g + (r & 3);
          st[mb][r] = (key <= rowpos) ? st[mb][r] : -INFINITY;
        }
    }
    float rmax = st[0][0];
#pragma unroll
    for (int mb = 0; mb < 2; ++mb)
#pragma unroll
      for (int r = 0; r < 16; ++r) rmax = fmaxf(rmax, st[mb][r]);
    rmax = max_with_partner_half(rmax);
    const float tmax = rmax * c;
    const bool grow = tmax > m_run + kRescaleStep;
    if (__any(grow)) {
      const float m_new = grow ? tmax : m_run;
      const float alpha = grow ? fast_exp2(m_run - m_new) : 1.0f;
      m_run = m_new;
      l_run *= alpha;
#pragma unroll
      for (int db = 0; db < 4; ++db) oacc[db] *= alpha;
    }
    const float neg_m = (m_run == -INFINITY) ? 0.0f : -m_run;
    float psum = 0.0f;
#pragma unroll
    for (int cc = 0; cc < 4; ++cc) {
      const int mb = cc >> 1, r0 = 8 * (cc & 1);
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        const float p0 = fast_exp2(__builtin_fmaf(st[mb][r0 + 2 * w], c, neg_m));
        const float p1 = fast_exp2(__builtin_fmaf(st[mb][r0 + 2 * w + 1], c, neg_m));
        pk[cc][w] = Mfma<T>::pack2(p0, p1);
        psum += p0 + p1;
      }
    }
    l_run += psum;
  };

  // Phases, one workgroup barrier apart: group 0 runs matrix(0) | vector(0) |
  // matrix(1) | vector(1) ... matrix(n_tiles); group 1 runs the same sequence one
  // phase later.  One loop per group behind a scalar branch (the wave number goes
  // through readfirstlane so that the compiler knows a wave runs one of them
  // only; in a shared loop body it keeps the two groups' values apart and
  // runs out of registers).  A vector step has no LDS traffic, so it leaves the
  // operand requests for the next matrix step in flight across the barrier.
  constexpr std::integral_constant<int, 0> kGroup0;
  constexpr std::integral_constant<int, 1> kGroup1;
  if (__builtin_amdgcn_readfirstlane(grp) == 0) {
    prefetch_ring(0);
    matrix_step(kGroup0, 0);
    __builtin_amdgcn_s_barrier();
    for (uint32_t kt = 0; kt < n_tiles; ++kt) {
      vector_step(kt);
      prefetch_ring(kt + 1);
      __builtin_amdgcn_s_barrier();
      matrix_step(kGroup0, kt + 1);
      __builtin_amdgcn_s_barrier();
    }
  } else {
    prefetch_ring(0);
    __builtin_amdgcn_s_barrier();
    for (uint32_t kt = 0; kt < n_tiles; ++kt) {
      matrix_step(kGroup1, kt);
      __builtin_amdgcn_s_barrier();
      vector_step(kt);
      prefetch_ring(kt + 1);
      __builtin_amdgcn_s_barrier();
    }
    matrix_step(kGroup1, n_tiles);
  }


  if constexpr (SPLIT) {
    const float l = sum_with_partner_half(l_run);
    if (row_valid) {
      const size_t part = (((size_t)tok * p.batch_pitch + seq) * p.n_q_heads + head) * p.n_split + blockIdx.y;
      float* orow = p.part_o + part * kHeadDim;
#pragma unroll
      for (int db = 0; db < 4; ++db)
#pragma unroll
        for (int q4 = 0; q4 < 4; ++q4)
          *(f32x4*)(orow + 32 * db + 8 * q4 + 4 * g) =
              f32x4{oacc[db][4 * q4], oacc[db][4 * q4 + 1], oacc[db][4 * q4 + 2], oacc[db][4 * q4 + 3]};
      if (g == 0) *(float2*)(p.part_ml + part * 2) = float2{m_run, l};
    }
  } else {
    const float l = sum_with_partner_half(l_run);
    if (row_valid) {
      const float inv = 1.0f / l;
      uint16_t* orow =
          p.out + (size_t)tok * p.q_token_stride + ((size_t)seq * p.n_q_heads + head) * kHeadDim;
#pragma unroll
      for (int db = 0; db < 4; ++db)
#pragma unroll
        for (int q4 = 0; q4 < 4; ++q4) {
          u32x2 w;
          w[0] = Mfma<T>::pack2(oacc[db][4 * q4] * inv, oacc[db][4 * q4 + 1] * inv);
          w[1] = Mfma<T>::pack2(oacc[db][4 * q4 + 2] * inv, oacc[db][4 * q4 + 3] * inv);
          *(u32x2*)(orow + 32 * db + 8 * q4 + 4 * g) = w;
        }
      if (p.lse && g == 0)
        p.lse[((size_t)tok * p.batch_pitch + seq) * p.n_q_heads + head] =
            (m_run + fast_log2(l)) * kLn2;
    }
  }
}

// ---------------------------------------------------------------------------
// Few query rows per K/V plane: the short last chunk of a prompt (1 - 63 tokens x 24
// sequences on caches of thousands of tokens in the reference's serving loop,
// src/serving/start copy.rs:71-101).  The ping-pong kernel above is built for tiles that
// are re-used by thousands of rows and sit in L2; here every K/V byte is used once by at
// most 384 rows and the call is a stream from HBM, like the single-token kernel: with few
// rows what matters is bytes in flight, not MFMA issue.  One workgroup = 4, 8 or 12 waves x
// 32 query rows = all (token, head) pairs of one GQA group (row r of the plane = token
// r / group, head r % group), so a plane is read once; the key range is split over gridDim.y
// workgroups (36 KB of LDS each), which leave partial rows for prefill_merge_kernel as the
// split form of the kernel above does.  Chunks of 32 keys go memory -> registers -> LDS
// (double-buffered, one barrier a chunk, the next chunks' loads in flight during the MFMAs of
// this one); operands and soft-max as above.
// ---------------------------------------------------------------------------
constexpr int kSK = 32;                        // keys per compute step
constexpr int kStStagersMax = 8 * kWave;       // one 16-byte piece of K and of V each moves a whole chunk

// kStDepth = chunks of loads a workgroup keeps in flight, each in its own set of staging
// registers (16 KB a chunk).  The call is bound by bytes in flight: with one chunk a workgroup
// moves 16 KB per memory round trip, whatever else it does.  Two chunks and two workgroups
// per compute unit measured 4-12 % faster than one chunk and three workgroups (24 sequences
// on 8192 keys: 2 tokens 70.1 -> 67.1 us, 8 tokens 80.2 -> 73.0, 16 tokens 94.9 -> 91.2; 16
// tokens x 16 sequences 78.4 -> 68.6); three chunks no better than two.
constexpr int kStDepth = 2;
// WAVES = 4, 8 or 12 waves of 32 query rows each: up to 128, 256 or 384 rows of a plane (16, 32
// or 48 tokens of a sequence with eight heads a group).  Four waves leave room for two
// workgroups a compute unit; eight and twelve fill a unit with one.
template <typename T, int WAVES>
__global__ __launch_bounds__(WAVES * kWave, WAVES == 4 ? 2 : 1) void chunk_stream_kernel(PrefillKernelArgs p) {
  constexpr int DEPTH = kStDepth;
  constexpr int kThreads = WAVES * kWave;
  constexpr int kStagers = kThreads < kStStagersMax ? kThreads : kStStagersMax;  // threads that move K/V
  constexpr int kCK = kSK;                       // keys per staged chunk
  constexpr int kStKsHalves = kCK * kKsPitch;
  constexpr int kStVsHalves = kCK * kVsPitch;
  constexpr int kPieces = kCK * 16 / kStagers;   // 16-byte pieces of K (and of V) a staging thread moves per chunk
  constexpr int kPieceRows = kStagers / 16;      // rows between a thread's pieces
  static_assert(kPieces * kStagers == kCK * 16, "the staging threads must tile a chunk");
  __shared__ __attribute__((aligned(16))) uint16_t smem[2 * kStKsHalves + 2 * kStVsHalves];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int j = lane & 31, g = lane >> 5;
  const uint32_t seq = blockIdx.x / p.n_kv_heads, kvh = blockIdx.x % p.n_kv_heads;
  const uint32_t S = p.interval, P0 = p.position_index;
  const uint32_t kmax = P0 + S - 1;
  const uint32_t all_tiles = kmax / kBK + 1;
  const uint32_t kt0 = blockIdx.y * p.split_tiles;
  if (kt0 >= all_tiles) return;  // (prefill_merge_kernel derives the live splits the same way)
  const uint32_t n_tiles = min(all_tiles - kt0, p.split_tiles);
  const uint32_t k0 = kt0 * kBK;                                   // first key of this split
  const uint32_t n_chunks = (min(kmax + 1, k0 + n_tiles * kBK) - k0 + kCK - 1) / kCK;

  const uint32_t rows = S * p.group;                                // query rows of the plane, <= 32 WAVES
  const uint32_t r = 32 * wave + j;
  const bool row_valid = r < rows;
  const uint32_t rc = row_valid ? r : rows - 1;
  const uint32_t tok = rc / p.group, head = kvh * p.group + rc % p.group;
  const uint32_t rowpos = P0 + tok;
  // positions of the wave's first and last row: chunks past the last are skipped, chunks up to
  // the first need no mask
  const uint32_t wave_first_pos = P0 + min(32u * wave, rows - 1) / p.group;
  const uint32_t wave_last_pos = P0 + min(32u * wave + 31u, rows - 1) / p.group;
  const bool wave_has_rows = 32u * wave < rows;

  u32x4 qreg[8];
  {
    const uint16_t* qrow =
        p.q + (size_t)tok * p.q_token_stride + ((size_t)seq * p.n_q_heads + head) * kHeadDim;
#pragma unroll
    for (int s = 0; s < 8; ++s) {
      qreg[s] = load16(qrow + 16 * s + 8 * g);
      if (p.negate_q) qreg[s] ^= 0x80008000u;
    }
  }
  const float c = p.c;

  const size_t plane_at = seq_plane_offset(p.seq_offsets, p.kv_stride_seq, seq) + kvh * p.kv_stride_head;
  const uint16_t* kplane = p.k + plane_at;
  const uint16_t* vplane = p.v + plane_at;
  const uint32_t stride_pos = (uint32_t)p.kv_stride_pos;
  // staging: the first 256 or 512 threads move one 32 x 128 chunk of K and one of V, two or one
  // 16-byte pieces of each (rows ld_r + 16 i or row ld_r, columns 8 ld_c ..), through buffer loads
  // whose descriptor ends at the last visible key: rows beyond it read as zeros.
  const bool stager = kThreads == kStagers || __builtin_amdgcn_readfirstlane(wave) < kStagers / kWave;
  const int ld_c = tid & 15, ld_r = (tid >> 4) & (kPieceRows - 1);
  const uint64_t kplane_u = uniform64(kplane), vplane_u = uniform64(vplane);
  const uint32_t chunk_bytes = kCK * stride_pos * 2;
  const uint64_t valid_bytes = uniform_u64(((uint64_t)kmax * stride_pos + kHeadDim) * 2);
  const uint32_t piece_off0 = (ld_r * stride_pos + 8 * ld_c) * 2;
  const uint32_t piece_step = kPieceRows * stride_pos * 2;
  u32x4 stg[DEPTH][2 * kPieces];
  auto load_chunk = [&](uint32_t ck, u32x4 (&st)[2 * kPieces]) {  // ck relative to this split's first chunk; wave-uniform
    if (!stager) return;
    const uint64_t off = (uint64_t)k0 * stride_pos * 2 + (uint64_t)ck * chunk_bytes;
    const uint32_t left = bytes_left(valid_bytes, off);
    const __amdgpu_buffer_rsrc_t kr = __builtin_amdgcn_make_buffer_rsrc((void*)(kplane_u + off), 0, left, kBufferFlags);
    const __amdgpu_buffer_rsrc_t vr = __builtin_amdgcn_make_buffer_rsrc((void*)(vplane_u + off), 0, left, kBufferFlags);
#pragma unroll
    for (int i = 0; i < kPieces; ++i) {
      st[i] = __builtin_amdgcn_raw_buffer_load_b128(kr, piece_off0 + i * piece_step, 0, 2);   // 2: non-temporal, read once
      st[kPieces + i] = __builtin_amdgcn_raw_buffer_load_b128(vr, piece_off0 + i * piece_step, 0, 2);
    }
  };
  const uint32_t lds0 = (uint32_t)(uintptr_t)(LdsHalf*)smem;
  const uint32_t ks_store = lds0 + 2 * (ld_r * kKsPitch + 8 * ld_c);
  const uint32_t vs_store = lds0 + 2 * (2 * kStKsHalves + ld_r * kVsPitch + 8 * ld_c);
  auto store_chunk = [&](uint32_t buf, const u32x4 (&st)[2 * kPieces]) {
    if (!stager) return;
#pragma unroll
    for (int i = 0; i < kPieces; ++i) {
      *(LdsU32x4*)(ks_store + 2 * (buf * kStKsHalves + kPieceRows * i * kKsPitch)) = st[i];
      *(LdsU32x4*)(vs_store + 2 * (buf * kStVsHalves + kPieceRows * i * kVsPitch)) = st[kPieces + i];
    }
  };
  // operand addresses: as in the kernel above (K rows as the A operand of S^T = K.Q^T, V through
  // the transposing read as the A operand of O^T += V^T.P^T, keys in the order P is left in)
  const uint32_t k_read = lds0 + 2 * (j * kKsPitch + 8 * g);
  const uint32_t v_read = lds0 + 2 * (2 * kStKsHalves + (4 * g + ((lane & 15) >> 2)) * kVsPitch +
                                      16 * ((lane >> 4) & 1) + 4 * (lane & 3));

  float m_run = -INFINITY, l_run = 0.0f;
  f32x16 oacc[4];
#pragma unroll
  for (int db = 0; db < 4; ++db)
#pragma unroll
    for (int e = 0; e < 16; ++e) oacc[db][e] = 0.0f;

  auto compute = [&](uint32_t ck) __attribute__((always_inline)) {
    const uint32_t kb = k0 + ck * kCK;
    const uint32_t buf = ck & 1;
    if (wave_has_rows && kb <= wave_last_pos) {
      const uint32_t ks = k_read + 2 * buf * kStKsHalves;
      const uint32_t vs = v_read + 2 * buf * kStVsHalves;
      f32x16 st;
#pragma unroll
      for (int e = 0; e < 16; ++e) st[e] = 0.0f;
#pragma unroll
      for (int s = 0; s < 8; ++s) {
        const u32x4 a = *(const LdsU32x4*)(ks + 2 * 16 * s);
        st = Mfma<T>::m32x32x16(a, qreg[s], st);
      }
      if (kb + kSK - 1 > wave_first_pos) {  // chunk crosses the diagonal of some row of this wave
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const uint32_t key = kb + 8 * (e >> 2) + 4 * g + (e & 3);
          st[e] = (key <= rowpos) ? st[e] : -INFINITY;
        }
      }
      float rmax = st[0];
#pragma unroll
      for (int e = 1; e < 16; ++e) rmax = fmaxf(rmax, st[e]);
      rmax = max_with_partner_half(rmax);
      const float tmax = rmax * c;
      const bool grow = tmax > m_run + kRescaleStep;
      if (__any(grow)) {
        const float m_new = grow ? tmax : m_run;
        const float alpha = grow ? fast_exp2(m_run - m_new) : 1.0f;
        m_run = m_new;
        l_run *= alpha;
#pragma unroll
        for (int db = 0; db < 4; ++db) oacc[db] *= alpha;
      }
      const float neg_m = (m_run == -INFINITY) ? 0.0f : -m_run;
      float psum = 0.0f;
      u32x4 pk[2];
#pragma unroll
      for (int cc = 0; cc < 2; ++cc)
#pragma unroll
        for (int w = 0; w < 4; ++w) {
          const float p0 = fast_exp2(__builtin_fmaf(st[8 * cc + 2 * w], c, neg_m));
          const float p1 = fast_exp2(__builtin_fmaf(st[8 * cc + 2 * w + 1], c, neg_m));
          pk[cc][w] = Mfma<T>::pack2(p0, p1);
          psum += p0 + p1;
        }
      l_run += psum;
#pragma unroll
      for (int cc = 0; cc < 2; ++cc)
#pragma unroll
        for (int db = 0; db < 4; ++db) {
          const uint32_t at = vs + 2 * (16 * cc * kVsPitch + 32 * db);
          const i16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LdsI16x4*)at);
          const i16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LdsI16x4*)(at + 2 * 8 * kVsPitch));
          const u32x2 l2 = __builtin_bit_cast(u32x2, lo), h2 = __builtin_bit_cast(u32x2, hi);
          oacc[db] = Mfma<T>::m32x32x16(u32x4{l2[0], l2[1], h2[0], h2[1]}, pk[cc], oacc[db]);
        }
    }
  };
  // chunk n travels through register set n % DEPTH; LDS is double-buffered by chunk parity
#pragma unroll
  for (int d = 0; d < DEPTH; ++d)
    if ((uint32_t)d < n_chunks) load_chunk(d, stg[d]);
  store_chunk(0, stg[0]);
  if ((uint32_t)DEPTH < n_chunks) load_chunk(DEPTH, stg[0]);
  __syncthreads();
  for (uint32_t ck0 = 0; ck0 < n_chunks; ck0 += DEPTH) {
#pragma unroll
    for (int u = 0; u < DEPTH; ++u) {
      const uint32_t ck = ck0 + u;
      if (ck < n_chunks) {  // (uniform over the workgroup: the barrier below is reached by all or none)
        compute(ck);
        if (ck + 1 < n_chunks) {
          const int set = (u + 1) % DEPTH;
          store_chunk((ck & 1) ^ 1, stg[set]);
          if (ck + 1 + DEPTH < n_chunks) load_chunk(ck + 1 + DEPTH, stg[set]);
        }
        __syncthreads();
      }
    }
  }

  const float l = sum_with_partner_half(l_run);
  if (!row_valid) return;
  if (p.n_split > 1) {
    const size_t part = (((size_t)tok * p.batch_pitch + seq) * p.n_q_heads + head) * p.n_split + blockIdx.y;
    float* orow = p.part_o + part * kHeadDim;
#pragma unroll
    for (int db = 0; db < 4; ++db)
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4)
        *(f32x4*)(orow + 32 * db + 8 * q4 + 4 * g) =
            f32x4{oacc[db][4 * q4], oacc[db][4 * q4 + 1], oacc[db][4 * q4 + 2], oacc[db][4 * q4 + 3]};
    if (g == 0) *(float2*)(p.part_ml + part * 2) = float2{m_run, l};
  } else {
    const float inv = 1.0f / l;
    uint16_t* orow =
        p.out + (size_t)tok * p.q_token_stride + ((size_t)seq * p.n_q_heads + head) * kHeadDim;
#pragma unroll
    for (int db = 0; db < 4; ++db)
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {
        u32x2 w;
        w[0] = Mfma<T>::pack2(oacc[db][4 * q4] * inv, oacc[db][4 * q4 + 1] * inv);
        w[1] = Mfma<T>::pack2(oacc[db][4 * q4 + 2] * inv, oacc[db][4 * q4 + 3] * inv);
        *(u32x2*)(orow + 32 * db + 8 * q4 + 4 * g) = w;
      }
    if (p.lse && g == 0)
      p.lse[((size_t)tok * p.batch_pitch + seq) * p.n_q_heads + head] = (m_run + fast_log2(l)) * kLn2;
  }
}

// Folds the partial results of a split launch: G lanes per (query row, four columns) take
// the row's splits in turn and combine through lane exchanges (with hundreds of splits and
// few rows a thread walking them alone would be one long chain of memory round trips).
// A row's live splits are those whose first tile is at or before the last key any row of
// its workgroup sees, as in the kernel above; a split whose keys are all masked for this row
// left (max = -inf, sum = 0) and weighs nothing.  Split 0 always holds key 0, so the maximum
// is finite.
template <typename T, int G>
__global__ __launch_bounds__(256) void prefill_merge_kernel(PrefillKernelArgs p, uint32_t batch) {
  const uint32_t quads = kHeadDim / 4;
  const size_t items = (size_t)p.interval * batch * p.n_q_heads * quads;
  const size_t gid = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const uint32_t sub = gid % G;
  const bool valid = gid / G < items;
  const size_t item = valid ? gid / G : 0;  // idle groups keep their lanes in the exchanges
  const uint32_t dq = item % quads;
  size_t r = item / quads;
  const uint32_t head = r % p.n_q_heads;
  r /= p.n_q_heads;
  const uint32_t seq = r % batch;
  const uint32_t tok = r / batch;
  const uint32_t wg_tokens = 32 * p.tblocks_per_wg;
  const uint32_t wg_last_tok = min(p.interval, (tok / wg_tokens + 1) * wg_tokens) - 1;
  const uint32_t all_tiles = (p.position_index + wg_last_tok) / kBK + 1;
  const uint32_t live = (all_tiles + p.split_tiles - 1) / p.split_tiles;
  const size_t row = ((size_t)tok * p.batch_pitch + seq) * p.n_q_heads + head;
  const float* ml = p.part_ml + row * p.n_split * 2;
  const float* po = p.part_o + row * p.n_split * kHeadDim + 4 * dq;
  float m = -INFINITY;
  for (uint32_t s = sub; s < live; s += G) m = fmaxf(m, ml[2 * s]);
#pragma unroll
  for (int x = 1; x < G; x <<= 1) m = fmaxf(m, __shfl_xor(m, x));
  float l = 0.0f;
  f32x4 o = {0.0f, 0.0f, 0.0f, 0.0f};
  for (uint32_t s = sub; s < live; s += G) {
    const float ms = ml[2 * s];
    const float w = (ms == -INFINITY) ? 0.0f : fast_exp2(ms - m);
    l += w * ml[2 * s + 1];
    o += w * *(const f32x4*)(po + (size_t)s * kHeadDim);
  }
#pragma unroll
  for (int x = 1; x < G; x <<= 1) {
    l += __shfl_xor(l, x);
#pragma unroll
    for (int e = 0; e < 4; ++e) o[e] += __shfl_xor(o[e], x);
  }
  if (!valid || sub != 0) return;
  const float inv = 1.0f / l;
  u32x2 w;
  w[0] = Mfma<T>::pack2(o[0] * inv, o[1] * inv);
  w[1] = Mfma<T>::pack2(o[2] * inv, o[3] * inv);
  *(u32x2*)(p.out + (size_t)tok * p.q_token_stride + ((size_t)seq * p.n_q_heads + head) * kHeadDim + 4 * dq) = w;
  if (p.lse && dq == 0) p.lse[row] = (m + fast_log2(l)) * kLn2;
}

uint32_t gcd_u32(uint32_t a, uint32_t b) {
  while (b) {
    const uint32_t t = a % b;
    a = b;
    b = t;
  }
  return a;
}

template <typename T>
hipError_t launch_pingpong(const AttnArgs& a, hipStream_t stream) {
  constexpr uint32_t kRowBlocks = kPpWaves;
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
  p.seq_offsets = a.seq_offsets;
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

  p.part_o = a.prefill_part_o;
  p.part_ml = a.prefill_part_ml;
  auto merge_launch = [&]() {
    const size_t items = (size_t)a.position_interval * a.batch * a.n_q_heads * (kHeadDim / 4);
    auto merge = [&](auto kernel, size_t lanes) {
      hipLaunchKernelGGL(kernel, dim3((uint32_t)((items * lanes + 255) / 256)), dim3(256), 0, stream, p, a.batch);
      return hipGetLastError();
    };
    // lanes per item: more when there are many splits to walk, as long as the grid stays small
    constexpr size_t kLanesMax = (size_t)1 << 21;
    if (p.n_split > 32 && items * 64 <= kLanesMax) return merge(prefill_merge_kernel<T, 64>, 64);
    if (p.n_split > 8 && items * 8 <= kLanesMax) return merge(prefill_merge_kernel<T, 8>, 8);
    return merge(prefill_merge_kernel<T, 1>, 1);
  };

  // Few query rows per plane on a cache long enough to be worth streaming: one workgroup
  // covers all rows of a GQA group, the key range is split until there are two
  // workgroups per compute unit (splits of at least 256 keys), as far as the workspace holds
  // the partial rows.
  const uint32_t all_tiles = (a.position_index + a.position_interval - 1) / kBK + 1;
  const size_t all_rows = (size_t)a.position_interval * a.batch_pitch * a.n_q_heads;
  const size_t plane_rows = (size_t)a.position_interval * a.group;
  if (plane_rows <= 384 && all_tiles >= 8) {
    const uint32_t planes = a.batch * a.n_kv_heads;
    // workgroups of four waves: two per compute unit (with one chunk in flight three were
    // better: see kStDepth); of eight or twelve waves: one.  Pieces of at least four tiles.
    const uint32_t waves = plane_rows <= 128 ? 4 : plane_rows <= 256 ? 8 : 12;
    const uint32_t slots = (waves == 4 ? 2 : 1) * a.n_cu;
    const size_t room = a.prefill_part_o ? a.prefill_part_rows / all_rows : 1;
    // a workgroup's time per tile (us, measured on 24 sequences x 8192 keys), and what one more
    // partial row per query row costs: written and read once, at about 4 TB/s
    const double tile_us = waves == 8 ? 2.0 : 2.5;
    const double split_us = (double)a.position_interval * a.batch * a.n_q_heads * (kHeadDim + 2) * 8 / 4e6;
    const uint32_t max_split = (uint32_t)(room < 4096 ? room : 4096);
    if (waves == 4) {
      // Two workgroups share a compute unit's throughput, so a slot that opens early is not
      // spare capacity: equal pieces, never more workgroups than slots (24 sequences on 8192
      // keys, 2 / 8 tokens: 67.6 / 73.1 us; as 5 pieces of 25 tiles and one of 4: 70.1 / 78.9)
      uint32_t want = slots / planes;
      if (want > max_split) want = max_split;
      if (want > all_tiles / 4) want = all_tiles / 4;
      if (want < 1) want = 1;
      p.split_tiles = (all_tiles + want - 1) / want;
      p.n_split = (all_tiles + p.split_tiles - 1) / p.split_tiles;
    } else {
      const KeySplit ks = plan_key_split(all_tiles, planes, slots, 4, max_split, split_us / tile_us);
      p.split_tiles = ks.split_tiles;
      p.n_split = ks.n_split;
    }
    // enough workgroups to be worth it (a lone sequence with one split would leave the part idle)
    if ((size_t)planes * p.n_split * 2 >= a.n_cu || planes * p.n_split >= p.combos * p.n_wg_tokens) {
      p.tblocks_per_wg = (a.position_interval + 31) / 32;  // (the merge derives every row's live splits from the chunk's last token)
      const dim3 grid(planes, p.n_split);
      if (waves == 4)
        hipLaunchKernelGGL((chunk_stream_kernel<T, 4>), grid, dim3(4 * kWave), 0, stream, p);
      else if (waves == 8)
        hipLaunchKernelGGL((chunk_stream_kernel<T, 8>), grid, dim3(8 * kWave), 0, stream, p);
      else
        hipLaunchKernelGGL((chunk_stream_kernel<T, 12>), grid, dim3(12 * kWave), 0, stream, p);
      const hipError_t e = hipGetLastError();
      if (e != hipSuccess || p.n_split == 1) return e;
      return merge_launch();
    }
  }

  uint32_t n_wg;
  if (p.xcd_mode) {
    const uint32_t per = 8 / p.combos;
    n_wg = 8 * ((p.n_wg_tokens + per - 1) / per);
  } else {
    n_wg = p.combos * p.n_wg_tokens;
  }
  // Few row blocks on a long cache: split the key range over more workgroups, as far as the
  // workspace holds the partial rows (plan_key_split weighs the longest chain of pieces a
  // compute unit runs against the partial rows every piece adds).
  p.n_split = 1;
  p.split_tiles = 0;
  const uint32_t base = p.combos * p.n_wg_tokens;
  const uint32_t max_tiles = (a.position_index + a.position_interval - 1) / kBK + 1;
  const size_t rows = (size_t)a.position_interval * a.batch_pitch * a.n_q_heads;
  // Only while the unsplit launch leaves at least half of the compute units idle: with more
  // of them busy the part runs this kernel at its power limit, idle units or not, and a split
  // only adds the partial rows (64 tokens x 24 sequences on 8192 keys, 192 workgroups: 229 us
  // unsplit, 235 us as pieces of 97 + 32 tiles on all 256 units).
  if (a.prefill_part_o && 2 * base <= a.n_cu && max_tiles >= 16) {
    // pieces of at least eight tiles (each pays the pipeline's first and last step); 1.9 us a
    // tile and workgroup (measured, 64 tokens x 24 sequences on 8192 keys)
    const size_t room = a.prefill_part_rows / rows;
    const double split_us = (double)a.position_interval * a.batch * a.n_q_heads * (kHeadDim + 2) * 8 / 4e6;
    const KeySplit ks = plan_key_split(max_tiles, base, a.n_cu, 8, (uint32_t)(room < 4096 ? room : 4096),
                                       split_us / 1.9);
    if (ks.n_split > 1) {
      p.split_tiles = ks.split_tiles;
      p.n_split = ks.n_split;
    }
  }
  if (p.n_split <= 1) {
    p.n_split = 1;
    hipLaunchKernelGGL((prefill_pingpong_kernel<T, false>), dim3(n_wg), dim3(kPpThreads), 0, stream, p);
    return hipGetLastError();
  }
  hipLaunchKernelGGL((prefill_pingpong_kernel<T, true>), dim3(n_wg, p.n_split), dim3(kPpThreads), 0, stream, p);
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) return e;
  return merge_launch();
}

}  // namespace

// Partial rows (128 + 2 floats each) a handle keeps for calls whose key range is split: 256
// splits of every row it can be asked for, at most 512 per compute unit (68 MB on 256 units).
size_t prefill_workspace_rows(uint32_t max_interval, uint32_t batch_capacity, uint32_t n_q_heads,
                              uint32_t n_cu) {
  if (max_interval < 2) return 0;  // single-token calls take the other kernel
  const size_t rows = (size_t)max_interval * batch_capacity * n_q_heads;
  const size_t cap = (size_t)512 * n_cu;
  return rows * 256 < cap ? rows * 256 : cap;
}

hipError_t launch_prefill(const AttnArgs& a, hipStream_t stream) {
  if (a.dtype == 0) return launch_pingpong<F16>(a, stream);
  return launch_pingpong<BF16>(a, stream);
}

}  // namespace ellm
