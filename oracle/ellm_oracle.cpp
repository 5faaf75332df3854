// TEST INFRASTRUCTURE ONLY.
//
// CPU restatement of the attention path of lucienhuangfu/eLLM (a CPU-only Rust
// crate that cannot be compiled without a nightly Rust toolchain).  It exists to
// check the HIP kernels and to serve as the timed CPU baseline; nothing in the
// shipped library links to, loads or calls this file.
//
// Arithmetic contract: K/V/Q/O are stored as IEEE binary16, bfloat16 or binary32;
// every intermediate (dot product, running max, denominator, output row) is
// binary32, as the operator's numerical contract states ("fp32 accumulation on
// both sides").  The all-f16 accumulation order of the reference's AVX-512 path
// (f16 FMA lanes + _mm512_reduce_add_ph + f16::exp) is NOT reproduced: that
// bit-level behaviour is "parity unpinned" and outside the contract.
//
// Reference anchors (paths relative to the reference tree):
//   oracle_dot_product              src/kernel/generic/flash_attention.rs:17-28
//   oracle_scalar_vector_mul_and_acc src/kernel/generic/flash_attention.rs:39-47
//   oracle_flash_attention_row      src/kernel/x86_64/f16_512/flash_attention.rs:30-92
//                                   (recurrence and scale placement; the generic
//                                   form at src/kernel/generic/flash_attention.rs:60-89
//                                   uses the unscaled score in one exponent, line 76,
//                                   which is a defect and is not followed)
//   oracle_assign                   src/compiler/assign.rs:11-38
//   oracle_attention_run            src/compiler/mul/attention.rs:83-153 (commented
//                                   body) with kv head = q head / group size and a
//                                   K/V base that does not move with position_index
//   oracle_barrier_*                src/runtime/barrier.rs:24-40
//   oracle_attention_run_threads    src/serving/start.rs:59-77 (one thread per core,
//                                   every thread calls run, then the barrier)
//   oracle_scale_softmax            known answer held in src/kernel/test.rs:605-629
//   oracle_schedule_calls           src/serving/start copy.rs:71-111 (the prompt in chunks of
//                                   sequence_chunk_size, a shorter last chunk, then one token
//                                   at a time); the prototype's loop runs the last chunk
//                                   twice and underflows on an empty prompt, which is not
//                                   followed
//   oracle_rms_norm                 src/kernel/generic/rms_norm.rs:6-26 (weight 1; eps is
//                                   added to the root mean square, not under the root)
//   oracle_complex_mul              src/kernel/generic/complex_mul.rs:3-20 (interleaved
//                                   (re, im) pairs; rotary table rows are (cos, sin) pairs)
//   oracle_norm_rope_row            src/kernel/x86_64/f16_512/matmul_rms_complex.rs:76-96 and
//                                   src/compiler/mul/matmul3.rs:482-491 (RMS norm then rotation
//                                   of one 128-wide head row, in place)
//   oracle_kv_append_norm_rope      the cache write the reference only hints at
//                                   (output_to_kv, src/compiler/zip_map/complex_zip.rs:92-100:
//                                   destination advanced by the position, rotary row advanced
//                                   by one head_size per position): key rows normalised and
//                                   rotated with the row of their position, value rows copied
//
//   oracle_matmul_nt / matmul3 /    src/compiler/mul/matmul3.rs:289-385 (three products, finalize
//   matmul_add                      of Q and K heads :243-254), src/compiler/mul/matmul_add.rs:
//                                   128-232 (residual + product); binary32 accumulation as in the
//                                   reference's own checks (matmul3.rs:553-570)
//
// Pins (checked in tests/test_oracle_*.py): the all-ones known answer, the 1*1+2*2
// literal, dot products 32 / 128 / 38, the 18-value scale_softmax literal, the
// assign literals, closed forms (position 0, equal scores, constant V, shift
// invariance), chunk invariance, a float64 two-pass brute force and torch SDPA;
// for the key-row path the 18-value rms_norm literal (rms_norm.rs:54-86), the
// 34-value complex_mul literal (complex_mul.rs:33-49), fused == separate calls
// (matmul_rms_complex.rs:215-322), closed forms (unit output RMS, zero row stays
// zero, rotations keep pair norms) and a float64 restatement; for the
// projections the input formulas of the reference's tests (src/ptensor/tensor.rs:1079-1230,
// src/compiler/mul/matmul3.rs:620-700) against a float64 numpy product, identity
// weights (the projection returns its input), linearity and the finalize of the pinned
// rms_norm / complex_mul.

#include <atomic>
#include <chrono>
#include <cmath>
#include <cstddef>
#include <cstdint>
#include <cstring>
#include <limits>
#include <thread>
#include <vector>

#if defined(__x86_64__)
#include <immintrin.h>
#endif
#if defined(__linux__)
#include <pthread.h>
#include <sched.h>
#endif

namespace {

// ---- storage types -------------------------------------------------------

enum Dtype : int { kF16 = 0, kBF16 = 1, kF32 = 2 };

inline float half_bits_to_float(uint16_t h) {
  const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1fu;
  uint32_t man = h & 0x3ffu;
  uint32_t bits;
  if (exp == 0) {
    if (man == 0) {
      bits = sign;
    } else {  // subnormal: normalise
      int e = -1;
      do {
        man <<= 1;
        ++e;
      } while ((man & 0x400u) == 0);
      man &= 0x3ffu;
      bits = sign | ((uint32_t)(127 - 15 - e) << 23) | (man << 13);
    }
  } else if (exp == 31) {
    bits = sign | 0x7f800000u | (man << 13);
  } else {
    bits = sign | ((exp + 127 - 15) << 23) | (man << 13);
  }
  float f;
  std::memcpy(&f, &bits, 4);
  return f;
}

// round-to-nearest-even binary32 -> binary16
inline uint16_t float_to_half_bits(float f) {
  uint32_t x;
  std::memcpy(&x, &f, 4);
  const uint32_t sign = (x >> 16) & 0x8000u;
  x &= 0x7fffffffu;
  if (x >= 0x7f800000u) {  // inf / nan
    return (uint16_t)(sign | 0x7c00u | ((x > 0x7f800000u) ? 0x200u : 0u));
  }
  if (x >= 0x477ff000u) {  // rounds to >= 65520 -> inf
    return (uint16_t)(sign | 0x7c00u);
  }
  if (x < 0x33000001u) {  // < 2^-25 (or exactly 2^-25, ties to even -> 0)
    return (uint16_t)sign;
  }
  int exp = (int)(x >> 23) - 127;
  uint32_t man = (x & 0x7fffffu) | 0x800000u;
  int shift;
  if (exp < -14) {  // subnormal half
    shift = 13 + (-14 - exp);
    exp = -15;
  } else {
    shift = 13;
  }
  uint32_t half_man = man >> shift;
  const uint32_t rem = man & ((1u << shift) - 1u);
  const uint32_t halfway = 1u << (shift - 1);
  if (rem > halfway || (rem == halfway && (half_man & 1u))) ++half_man;
  // half_man carries the implicit bit for normals: adding the exponent field
  // below lets a mantissa overflow carry into the exponent naturally.
  uint32_t out;
  if (exp == -15) {
    out = half_man;  // subnormal (or rounds up into the smallest normal)
  } else {
    out = ((uint32_t)(exp + 15) << 10) + (half_man - 0x400u);
  }
  return (uint16_t)(sign | out);
}

inline float bf16_bits_to_float(uint16_t h) {
  uint32_t bits = (uint32_t)h << 16;
  float f;
  std::memcpy(&f, &bits, 4);
  return f;
}

inline uint16_t float_to_bf16_bits(float f) {
  uint32_t x;
  std::memcpy(&x, &f, 4);
  if ((x & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((x >> 16) | 0x40u);
  const uint32_t lsb = (x >> 16) & 1u;
  x += 0x7fffu + lsb;
  return (uint16_t)(x >> 16);
}

inline size_t dtype_size(int dt) { return dt == kF32 ? 4 : 2; }

inline float load_elem(const void* p, size_t i, int dt) {
  switch (dt) {
    case kF16:
      return half_bits_to_float(((const uint16_t*)p)[i]);
    case kBF16:
      return bf16_bits_to_float(((const uint16_t*)p)[i]);
    default:
      return ((const float*)p)[i];
  }
}

inline void store_elem(void* p, size_t i, int dt, float v) {
  switch (dt) {
    case kF16:
      ((uint16_t*)p)[i] = float_to_half_bits(v);
      break;
    case kBF16:
      ((uint16_t*)p)[i] = float_to_bf16_bits(v);
      break;
    default:
      ((float*)p)[i] = v;
  }
}

inline const void* elem_ptr(const void* base, size_t elems, int dt) {
  return (const char*)base + elems * dtype_size(dt);
}
inline void* elem_ptr(void* base, size_t elems, int dt) {
  return (char*)base + elems * dtype_size(dt);
}

#if defined(__x86_64__)
// Hardware binary16 -> binary32 (exact, so identical to the bit routine above);
// only taken when the host CPU reports F16C.
__attribute__((target("f16c,avx"))) void load_row_f16_hw(const uint16_t* src, float* dst, size_t n) {
  size_t i = 0;
  for (; i + 8 <= n; i += 8) {
    __m128i h = _mm_loadu_si128((const __m128i*)(src + i));
    _mm256_storeu_ps(dst + i, _mm256_cvtph_ps(h));
  }
  for (; i < n; ++i) dst[i] = half_bits_to_float(src[i]);
}
const bool g_have_f16c = __builtin_cpu_supports("f16c") && __builtin_cpu_supports("avx");
#else
const bool g_have_f16c = false;
#endif

// Decode one stored row into binary32 (exact for all three storage types).
inline void load_row(const void* base, size_t elems, int dt, float* dst, size_t n) {
#if defined(__x86_64__)
  if (dt == kF16 && g_have_f16c) {
    load_row_f16_hw((const uint16_t*)base + elems, dst, n);
    return;
  }
#endif
  for (size_t i = 0; i < n; ++i) dst[i] = load_elem(base, elems + i, dt);
}

// ---- leaf helpers ---------------------------------------------------------

// src/kernel/generic/flash_attention.rs:17-28 — sequential sum from a zero start.
inline float dot_product(const float* a, const float* b, size_t n) {
  float r = 0.0f;
  for (size_t i = 0; i < n; ++i) r = r + a[i] * b[i];
  return r;
}

// src/kernel/generic/flash_attention.rs:39-47 — o[i] = s1*o[i] + s2*v[i].
inline void scalar_vector_mul_and_acc(float s1, float* o, float s2, const float* v, size_t n) {
  for (size_t i = 0; i < n; ++i) o[i] = s1 * o[i] + s2 * v[i];
}

// src/kernel/generic/rms_norm.rs:6-26 — sequential sum of squares, mean, then
// 1 / (sqrt(mean) + eps); no weight vector.
inline void rms_norm(const float* in, float* out, size_t n, float eps) {
  float sum = in[0] * in[0];
  for (size_t i = 1; i < n; ++i) sum = sum + in[i] * in[i];
  const float variance = sum / (float)n;
  const float rrms = 1.0f / (std::sqrt(variance) + eps);
  for (size_t i = 0; i < n; ++i) out[i] = in[i] * rrms;
}

// src/kernel/generic/complex_mul.rs:3-20 — (a + ib)(c + id) on interleaved pairs.
inline void complex_mul(const float* x, const float* y, float* out, size_t n) {
  for (size_t i = 0; i + 1 < n; i += 2) {
    const float a = x[i], b = x[i + 1], c = y[i], d = y[i + 1];
    const float e = a * c - b * d;
    const float f = a * d + b * c;
    out[i] = e;
    out[i + 1] = f;
  }
}

// One query row against keys 0..=position of one K/V plane.
// src/kernel/x86_64/f16_512/flash_attention.rs:47-86: m starts at -inf, d at 0,
// the output row at 0 and stays normalised after every key; the score is scaled
// before it is used anywhere.
void flash_attention_row(const void* q, const void* K, const void* V, void* o, float* lse,
                         float inverse_sqrt_head, size_t length, size_t stride,
                         size_t position, int dt) {
  std::vector<float> qf(length), kf(length), vf(length), acc(length, 0.0f);
  load_row(q, 0, dt, qf.data(), length);
  float m_prev = -std::numeric_limits<float>::infinity();
  float d_prev = 0.0f;
  size_t offset = 0;
  for (size_t i = 0; i <= position; ++i) {
    load_row(K, offset, dt, kf.data(), length);
    load_row(V, offset, dt, vf.data(), length);
    float x = dot_product(qf.data(), kf.data(), length);
    x = x * inverse_sqrt_head;
    const float m = (x > m_prev) ? x : m_prev;
    const float update_exp = d_prev * std::exp(m_prev - m);
    const float add_exp = std::exp(x - m);
    const float d = update_exp + add_exp;
    const float u = update_exp / d;
    const float a = add_exp / d;
    scalar_vector_mul_and_acc(u, acc.data(), a, vf.data(), length);
    m_prev = m;
    d_prev = d;
    offset += stride;
  }
  for (size_t i = 0; i < length; ++i) store_elem(o, i, dt, acc[i]);
  if (lse) *lse = m_prev + std::log(d_prev);
}

// src/compiler/assign.rs:11-38
bool assign(size_t length, size_t num, size_t id, size_t* begin, size_t* end) {
  if (length < id + 1) return false;
  const size_t quotient = length / num, remainder = length % num;
  if (remainder == 0) {
    *begin = quotient * id;
    *end = *begin + quotient;
    return true;
  }
  if (id < remainder) {
    *begin = (quotient + 1) * id;
    *end = *begin + quotient + 1;
    return true;
  }
  *begin = quotient * id + remainder;
  *end = *begin + quotient;
  return true;
}

// src/runtime/barrier.rs:7-40 — sense-reversing spin barrier.
struct alignas(64) PaddedAtomic {
  std::atomic<size_t> v{0};
};
struct Barrier {
  PaddedAtomic arrived, generation;
  size_t tids;
  explicit Barrier(size_t n) : tids(n) {}
  void wait() {
    const size_t gen = generation.v.load(std::memory_order_relaxed);
    const size_t n = arrived.v.fetch_add(1, std::memory_order_acq_rel) + 1;
    if (n == tids) {
      arrived.v.store(0, std::memory_order_relaxed);
      generation.v.store(gen + 1, std::memory_order_release);
      return;
    }
    while (generation.v.load(std::memory_order_acquire) == gen) {
#if defined(__x86_64__)
      __builtin_ia32_pause();
#endif
    }
  }
};

// src/serving/start.rs:43-61 pins worker i to core i (core_affinity::set_for_current).  Here:
// the i-th core of the set the process was allowed to run on when the pool started, so
// that a process confined to a share of a machine pins inside its share.
struct CoreSet {
  std::vector<int> cores;
  CoreSet() {
#if defined(__linux__)
    cpu_set_t set;
    CPU_ZERO(&set);
    if (sched_getaffinity(0, sizeof(set), &set) == 0)
      for (int c = 0; c < CPU_SETSIZE; ++c)
        if (CPU_ISSET(c, &set)) cores.push_back(c);
#endif
  }
  void pin_current(size_t tid) const {
#if defined(__linux__)
    if (cores.empty()) return;
    cpu_set_t set;
    CPU_ZERO(&set);
    CPU_SET(cores[tid % cores.size()], &set);
    pthread_setaffinity_np(pthread_self(), sizeof(set), &set);
#else
    (void)tid;
#endif
  }
};

}  // namespace

extern "C" {

// Operator description: the fields of compiler::mul::attention::Attention
// (src/compiler/mul/attention.rs:12-27) plus the storage type and an optional
// log-sum-exp output [position_interval][capacity][heads] in binary32.
struct ellm_oracle_attn {
  const void* q;
  const void* k;
  const void* v;
  void* out;
  float* lse;  // may be null
  size_t batch_capacity;
  size_t attention_head_num;
  size_t kv_head_num;
  size_t head_size;
  size_t kv_strides[4];  // elements: sequence slot, kv head, position, 1
  float inverse_sqrt_head;
  int dtype;
};

float ellm_oracle_dot_product_f32(const float* a, const float* b, size_t n) {
  return dot_product(a, b, n);
}

void ellm_oracle_scalar_vector_mul_and_acc_f32(float s1, float* o, float s2, const float* v,
                                               size_t n) {
  scalar_vector_mul_and_acc(s1, o, s2, v, n);
}

// softmax(scale * x); known answer in src/kernel/test.rs:605-629.
void ellm_oracle_scale_softmax_f32(const float* x, float* out, size_t n, float scale) {
  float m = -std::numeric_limits<float>::infinity();
  for (size_t i = 0; i < n; ++i) m = std::fmax(m, x[i] * scale);
  float d = 0.0f;
  for (size_t i = 0; i < n; ++i) {
    out[i] = std::exp(x[i] * scale - m);
    d += out[i];
  }
  for (size_t i = 0; i < n; ++i) out[i] /= d;
}

void ellm_oracle_flash_attention(const void* q, const void* K, const void* V, void* o, float* lse,
                                 float inverse_sqrt_head, size_t length, size_t stride,
                                 size_t position, int dtype) {
  flash_attention_row(q, K, V, o, lse, inverse_sqrt_head, length, stride, position, dtype);
}

int ellm_oracle_assign(size_t length, size_t num, size_t id, size_t* begin, size_t* end) {
  return assign(length, num, id, begin, end) ? 1 : 0;
}

// One thread's share of Attention::run.  Tasks are (token in chunk, sequence,
// query head) with the query head varying fastest; Q and O live at
// ((token*batch_capacity + sequence)*heads + head)*head_size.
// `positions` (may be null) gives a per-sequence position for single-token
// steps whose sequences have different lengths; the reference has one shared
// position_index only.
int ellm_oracle_attention_run(const ellm_oracle_attn* op, size_t position_index,
                              size_t position_interval, size_t batch_size,
                              const uint32_t* positions, size_t cpu_num, size_t thread_id) {
  if (!op || op->kv_head_num == 0 || op->attention_head_num % op->kv_head_num != 0) return 1;
  if (batch_size > op->batch_capacity || cpu_num == 0 || thread_id >= cpu_num) return 1;
  if (positions && position_interval != 1) return 1;
  const size_t heads = op->attention_head_num;
  const size_t group = heads / op->kv_head_num;
  const size_t stride = batch_size * heads;
  size_t begin, end;
  if (!assign(position_interval * stride, cpu_num, thread_id, &begin, &end)) return 0;
  const size_t max_stride = op->batch_capacity * heads;
  size_t high = begin / stride;
  size_t rem = begin % stride;
  size_t row = rem / heads, col = rem % heads;
  for (size_t t = begin; t < end; ++t) {
    const size_t index = (high * max_stride + row * heads + col) * op->head_size;
    const size_t kv_head = col / group;
    const size_t kv_index = row * op->kv_strides[0] + kv_head * op->kv_strides[1];
    const size_t position = positions ? (size_t)positions[row] : position_index + high;
    float* lse = op->lse ? op->lse + (high * max_stride + row * heads + col) : nullptr;
    flash_attention_row(elem_ptr(op->q, index, op->dtype), elem_ptr(op->k, kv_index, op->dtype),
                        elem_ptr(op->v, kv_index, op->dtype), elem_ptr(op->out, index, op->dtype),
                        lse, op->inverse_sqrt_head, op->head_size, op->kv_strides[2], position,
                        op->dtype);
    if (++col == heads) {
      col = 0;
      if (++row == batch_size) {
        row = 0;
        ++high;
      }
    }
  }
  return 0;
}

// The serving loop's shape (src/serving/start.rs:43-77): one thread per core,
// optionally pinned, each calls run() for its id and then meets the barrier.
// Returns wall seconds measured on the calling thread around spawn..join of
// `repeats` passes (threads are created once).
double ellm_oracle_attention_run_threads(const ellm_oracle_attn* op, size_t position_index,
                                         size_t position_interval, size_t batch_size,
                                         const uint32_t* positions, size_t n_threads, int pin,
                                         size_t repeats) {
  if (n_threads == 0) return -1.0;
  Barrier barrier(n_threads);
  std::atomic<int> err{0};
  std::vector<std::thread> pool;
  const CoreSet cores;
  const auto t0 = std::chrono::steady_clock::now();
  for (size_t tid = 0; tid < n_threads; ++tid) {
    pool.emplace_back([&, tid]() {
      if (pin) cores.pin_current(tid);
      for (size_t r = 0; r < repeats; ++r) {
        if (ellm_oracle_attention_run(op, position_index, position_interval, batch_size, positions,
                                      n_threads, tid))
          err.store(1);
        barrier.wait();
      }
    });
  }
  for (auto& t : pool) t.join();
  const auto t1 = std::chrono::steady_clock::now();
  if (err.load()) return -1.0;
  return std::chrono::duration<double>(t1 - t0).count();
}

// Selected (token, sequence, head) rows only: the bounded sample used when the
// full problem is too large for the CPU.  rows = n triples (token_in_chunk,
// sequence, head).  Work is split over threads by the same assign().  `positions` (may be
// null) gives per-sequence positions as in ellm_oracle_attention_run; `pin` pins thread i
// to the i-th core the process may run on.
double ellm_oracle_attention_rows_threads_ex(const ellm_oracle_attn* op, size_t position_index,
                                             const uint32_t* positions, const uint32_t* rows,
                                             size_t n_rows, void* out_rows, float* lse_rows,
                                             size_t n_threads, int pin) {
  if (!op || n_threads == 0) return -1.0;
  const size_t heads = op->attention_head_num;
  const size_t group = heads / op->kv_head_num;
  const size_t max_stride = op->batch_capacity * heads;
  std::vector<std::thread> pool;
  const CoreSet cores;
  const auto t0 = std::chrono::steady_clock::now();
  for (size_t tid = 0; tid < n_threads; ++tid) {
    pool.emplace_back([&, tid]() {
      if (pin) cores.pin_current(tid);
      size_t begin, end;
      if (!assign(n_rows, n_threads, tid, &begin, &end)) return;
      for (size_t r = begin; r < end; ++r) {
        const size_t high = rows[3 * r], row = rows[3 * r + 1], col = rows[3 * r + 2];
        const size_t index = (high * max_stride + row * heads + col) * op->head_size;
        const size_t kv_index = row * op->kv_strides[0] + (col / group) * op->kv_strides[1];
        const size_t position = positions ? (size_t)positions[row] : position_index + high;
        flash_attention_row(elem_ptr(op->q, index, op->dtype),
                            elem_ptr(op->k, kv_index, op->dtype),
                            elem_ptr(op->v, kv_index, op->dtype),
                            elem_ptr(out_rows, r * op->head_size, op->dtype),
                            lse_rows ? lse_rows + r : nullptr, op->inverse_sqrt_head,
                            op->head_size, op->kv_strides[2], position, op->dtype);
      }
    });
  }
  for (auto& t : pool) t.join();
  const auto t1 = std::chrono::steady_clock::now();
  return std::chrono::duration<double>(t1 - t0).count();
}

double ellm_oracle_attention_rows_threads(const ellm_oracle_attn* op, size_t position_index,
                                          const uint32_t* rows, size_t n_rows, void* out_rows,
                                          float* lse_rows, size_t n_threads) {
  return ellm_oracle_attention_rows_threads_ex(op, position_index, nullptr, rows, n_rows, out_rows,
                                               lse_rows, n_threads, 0);
}

void ellm_oracle_rms_norm_f32(const float* in, float* out, size_t n, float eps) {
  rms_norm(in, out, n, eps);
}
void ellm_oracle_complex_mul_f32(const float* x, const float* y, float* out, size_t n) {
  complex_mul(x, y, out, n);
}

// RMS norm then rotation of one stored row, both in binary32, rounded to the
// storage type once at the end (the reference's all-f16 path rounds after every
// operation; like its accumulation order that is outside the contract).
void ellm_oracle_norm_rope_row(const void* row, const void* rope_row, void* out, size_t n,
                               float eps, int dtype) {
  std::vector<float> x(n), r(n), y(n);
  load_row(row, 0, dtype, x.data(), n);
  load_row(rope_row, 0, dtype, r.data(), n);
  rms_norm(x.data(), y.data(), n, eps);
  complex_mul(y.data(), r.data(), x.data(), n);
  for (size_t i = 0; i < n; ++i) store_elem(out, i, dtype, x[i]);
}

// Cache write with the key rows normalised and rotated.  Sources are
// [n_tokens][src_batch_pitch][kv_heads][head_size]; the cache layer is
// [sequences][kv_heads][capacity][head_size]; rope is [positions][head_size].
// Token t of sequence b lands at position (positions ? positions[b] : position_index) + t
// and its key is rotated with that position's row.  Returns 0, or 1 when a
// position falls outside the cache or the table (nothing is written then).
int ellm_oracle_kv_append_norm_rope(void* k_cache, void* v_cache, size_t kv_heads, size_t capacity,
                                    size_t head_size, size_t position_index, size_t n_tokens,
                                    size_t batch_size, const void* k_src, const void* v_src,
                                    size_t src_batch_pitch, const void* rope, size_t rope_positions,
                                    float eps, const uint32_t* positions, int dtype) {
  for (size_t b = 0; b < batch_size; ++b) {
    const size_t p0 = positions ? positions[b] : position_index;
    if (p0 + n_tokens > capacity || p0 + n_tokens > rope_positions) return 1;
  }
  const size_t esz = dtype_size(dtype);
  for (size_t t = 0; t < n_tokens; ++t)
    for (size_t b = 0; b < batch_size; ++b)
      for (size_t h = 0; h < kv_heads; ++h) {
        const size_t pos = (positions ? positions[b] : position_index) + t;
        const size_t src = ((t * src_batch_pitch + b) * kv_heads + h) * head_size;
        const size_t dst = ((b * kv_heads + h) * capacity + pos) * head_size;
        ellm_oracle_norm_rope_row(elem_ptr(k_src, src, dtype), elem_ptr(rope, pos * head_size, dtype),
                                  elem_ptr(k_cache, dst, dtype), head_size, eps, dtype);
        std::memcpy(elem_ptr(v_cache, dst, dtype), elem_ptr(v_src, src, dtype), head_size * esz);
      }
  return 0;
}

// ---- projections either side of attention ----------------------------------------
// C[m][n] = sum_k a[m][k] * b_nt[n][k], binary32 accumulation in ascending k: the
// arithmetic of the reference's own checks (gemm_ref_f16_acc_f32_from_wnt,
// src/compiler/mul/matmul3.rs:553-570; verify_matmul_nt, src/ptensor/tensor.rs:1202-1228).
// The reference's AVX-512 micro-kernel accumulates in binary16 per 3x32 tile
// (src/kernel/x86_64/f16_512/matmul_rms_complex.rs:24-66), which is outside the contract.
void ellm_oracle_matmul_nt(const void* a, const void* b_nt, float* c, size_t m, size_t n, size_t k,
                           int dtype) {
  std::vector<float> arow(k), brow(k);
  for (size_t i = 0; i < m; ++i) {
    load_row(a, i * k, dtype, arow.data(), k);
    for (size_t jn = 0; jn < n; ++jn) {
      load_row(b_nt, jn * k, dtype, brow.data(), k);
      float sum = 0.0f;
      for (size_t kk = 0; kk < k; ++kk) sum += arow[kk] * brow[kk];
      c[i * n + jn] = sum;
    }
  }
}

// MatMul3::run (src/compiler/mul/matmul3.rs:289-385) over position_interval token rows:
// the three products, then per finished 128-wide head row of Q and K the finalize of
// :243-254 (rms_norm then complex_mul with a rotary row, eps from :436-451 passed in),
// all in binary32, one rounding at the end.  hidden: [interval][batch_pitch][k];
// q_state: [interval][batch_pitch][q_heads * head]; K/V rows go to
// state + sequence * kv_strides[0] + head * kv_strides[1] + position * kv_strides[2];
// rotary row of head h at position p: rope + p * rope_pos_stride + h * rope_head_stride
// (the reference: position stride 0, head stride head_size, :243-251).
// Returns 0, or 1 when a position falls outside capacity or the table.
int ellm_oracle_matmul3(const void* hidden, const void* wq, const void* wk, const void* wv,
                        void* q_state, void* k_state, void* v_state, const void* rope,
                        size_t rope_pos_stride, size_t rope_head_stride, size_t rope_elems,
                        size_t k, size_t batch_pitch, size_t batch_size, size_t q_heads,
                        size_t kv_heads, size_t head, const size_t* kv_strides, size_t capacity,
                        size_t position_index, size_t interval, const uint32_t* positions,
                        float eps, int dtype) {
  const size_t heads_max = q_heads > kv_heads ? q_heads : kv_heads;
  for (size_t b = 0; b < batch_size; ++b) {
    const size_t last = (positions ? positions[b] : position_index) + interval - 1;
    if (last >= capacity) return 1;
    if (last * rope_pos_stride + (heads_max - 1) * rope_head_stride + head > rope_elems) return 1;
  }
  std::vector<float> x(k), w(k), c(head), y(head), r(head), o(head);
  auto head_row = [&](const void* weights, size_t h) {
    for (size_t jn = 0; jn < head; ++jn) {
      load_row(weights, (h * head + jn) * k, dtype, w.data(), k);
      float sum = 0.0f;
      for (size_t kk = 0; kk < k; ++kk) sum += x[kk] * w[kk];
      c[jn] = sum;
    }
  };
  auto finalize = [&](size_t h, size_t pos) {
    load_row(rope, pos * rope_pos_stride + h * rope_head_stride, dtype, r.data(), head);
    rms_norm(c.data(), y.data(), head, eps);
    complex_mul(y.data(), r.data(), o.data(), head);
  };
  for (size_t t = 0; t < interval; ++t)
    for (size_t b = 0; b < batch_size; ++b) {
      const size_t row = t * batch_pitch + b;
      const size_t pos = (positions ? positions[b] : position_index) + t;
      load_row(hidden, row * k, dtype, x.data(), k);
      for (size_t h = 0; h < q_heads; ++h) {
        head_row(wq, h);
        finalize(h, pos);
        for (size_t i = 0; i < head; ++i) store_elem(q_state, (row * q_heads + h) * head + i, dtype, o[i]);
      }
      for (size_t h = 0; h < kv_heads; ++h) {
        const size_t dst = b * kv_strides[0] + h * kv_strides[1] + pos * kv_strides[2];
        head_row(wk, h);
        finalize(h, pos);
        for (size_t i = 0; i < head; ++i) store_elem(k_state, dst + i, dtype, o[i]);
        head_row(wv, h);
        for (size_t i = 0; i < head; ++i) store_elem(v_state, dst + i, dtype, c[i]);
      }
    }
  return 0;
}

// MatMulAdd::run (src/compiler/mul/matmul_add.rs:128-232): output = residual + a . b_nt^T
// (the reference copies the residual tile into the output and accumulates the product on
// top, :176-215), binary32, one rounding.  a: [interval][batch_pitch][k]; residual,
// output: [interval][batch_pitch][n].
void ellm_oracle_matmul_add(const void* a, const void* b_nt, const void* residual, void* output,
                            size_t n, size_t k, size_t batch_pitch, size_t batch_size,
                            size_t interval, int dtype) {
  std::vector<float> x(k), w(k);
  for (size_t t = 0; t < interval; ++t)
    for (size_t b = 0; b < batch_size; ++b) {
      const size_t row = t * batch_pitch + b;
      load_row(a, row * k, dtype, x.data(), k);
      for (size_t jn = 0; jn < n; ++jn) {
        load_row(b_nt, jn * k, dtype, w.data(), k);
        float sum = 0.0f;
        for (size_t kk = 0; kk < k; ++kk) sum += x[kk] * w[kk];
        store_elem(output, row * n + jn, dtype, load_elem(residual, row * n + jn, dtype) + sum);
      }
    }
}

// The (position_index, position_interval) pairs every operator of the graph is run with
// for one request.  src/serving/start copy.rs:71-86 computes the last chunk as
//   remainder = prompt_end % chunk;  last_interval = remainder ? remainder : chunk;
//   last_position = prompt_end - last_interval
// (stated there for prompt_begin = 0; lengths are taken from prompt_begin here), runs full
// chunks before it (:89-95), the last chunk (:97-101), then single tokens (:102-113).
// Returns the number of calls, or -1 when `capacity` pairs do not hold them.
long ellm_oracle_schedule_calls(size_t prompt_begin, size_t prompt_end, size_t chunk,
                                size_t generation_end, size_t* positions, size_t* intervals,
                                size_t capacity) {
  if (chunk == 0 || prompt_end < prompt_begin) return -1;
  size_t n = 0;
  auto push = [&](size_t pos, size_t interval) {
    if (n < capacity) {
      positions[n] = pos;
      intervals[n] = interval;
    }
    ++n;
  };
  if (prompt_end > prompt_begin) {
    const size_t remainder = (prompt_end - prompt_begin) % chunk;
    const size_t last_interval = remainder ? remainder : chunk;
    const size_t last_position = prompt_end - last_interval;
    for (size_t pos = prompt_begin; pos < last_position; pos += chunk) push(pos, chunk);
    push(last_position, last_interval);
  }
  for (size_t pos = prompt_end; pos < generation_end; ++pos) push(pos, 1);
  return n <= capacity ? (long)n : -1;
}

// Storage conversions exposed so tests can check them against numpy.
uint16_t ellm_oracle_f32_to_f16(float f) { return float_to_half_bits(f); }
float ellm_oracle_f16_to_f32(uint16_t h) { return half_bits_to_float(h); }
uint16_t ellm_oracle_f32_to_bf16(float f) { return float_to_bf16_bits(f); }
float ellm_oracle_bf16_to_f32(uint16_t h) { return bf16_bits_to_float(h); }

// Barrier self-check in the manner of src/runtime/barrier.rs:57-83: every
// thread increments a counter between barriers; returns 0 when no thread ever
// observes a count from the wrong phase.
int ellm_oracle_barrier_selftest(size_t n_threads, size_t rounds) {
  Barrier barrier(n_threads);
  std::atomic<size_t> counter{0};
  std::atomic<int> bad{0};
  std::vector<std::thread> pool;
  for (size_t tid = 0; tid < n_threads; ++tid) {
    pool.emplace_back([&]() {
      for (size_t r = 0; r < rounds; ++r) {
        counter.fetch_add(1);
        barrier.wait();
        if (counter.load() != (r + 1) * n_threads) bad.store(1);
        barrier.wait();
      }
    });
  }
  for (auto& t : pool) t.join();
  return bad.load();
}

}  // extern "C"
