// C ABI of the attention path (declared in include/ellm_attn.h): argument
// validation, the operator handle, the K/V cache object, error reporting.
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <new>

#include "../../include/ellm_attn.h"
#include "kernels.hpp"

namespace {

thread_local char g_error[512] = "";

int fail(int status, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return status;
}

int fail_hip(hipError_t e, const char* what) {
  return fail(ELLM_ERR_HIP, "%s: %s", what, hipGetErrorString(e));
}

bool aligned16(const void* p) { return ((uintptr_t)p & 15u) == 0; }

}  // namespace

int ellm::current_gfx950_device(int* device, int* n_cu) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) {
    (void)hipGetLastError();
    return fail(ELLM_ERR_NO_DEVICE, "hipGetDevice: %s", hipGetErrorString(e));
  }
  hipDeviceProp_t prop;
  e = hipGetDeviceProperties(&prop, dev);
  if (e != hipSuccess) return fail_hip(e, "hipGetDeviceProperties");
  if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
    return fail(ELLM_ERR_NO_DEVICE, "device %d is %s; this library carries gfx950 code only", dev,
                prop.gcnArchName);
  *device = dev;
  *n_cu = prop.multiProcessorCount;
  return ELLM_OK;
}

int ellm::check_current_device(int device) {
  int now = -1;
  const hipError_t e = hipGetDevice(&now);
  if (e != hipSuccess) return fail_hip(e, "hipGetDevice");
  if (now != device)
    return fail(ELLM_ERR_INVALID_ARGUMENT,
                "the handle was created on device %d; the calling thread's current device is %d",
                device, now);
  return ELLM_OK;
}

int ellm::set_error(int status, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return status;
}

int ellm::validate_attn_desc(const ellm_attn_desc* d) {
  if (!d) return fail(ELLM_ERR_INVALID_ARGUMENT, "null descriptor");
  if (!d->q || !d->k || !d->v || !d->out)
    return fail(ELLM_ERR_INVALID_ARGUMENT, "q, k, v and out must be non-null device pointers");
  if (!aligned16(d->q) || !aligned16(d->k) || !aligned16(d->v) || !aligned16(d->out))
    return fail(ELLM_ERR_INVALID_ARGUMENT, "q, k, v and out must be 16-byte aligned");
  if (d->dtype != ELLM_DTYPE_F16 && d->dtype != ELLM_DTYPE_BF16)
    return fail(ELLM_ERR_INVALID_ARGUMENT, "dtype %d is neither ELLM_DTYPE_F16 nor ELLM_DTYPE_BF16",
                d->dtype);
  if (d->head_size != 128)
    return fail(ELLM_ERR_UNSUPPORTED, "head_size %zu: only 128 is supported", d->head_size);
  if (d->batch_size == 0 || d->attention_head_num == 0 || d->kv_head_num == 0)
    return fail(ELLM_ERR_INVALID_ARGUMENT, "batch_size, attention_head_num, kv_head_num must be > 0");
  if (d->attention_head_num % d->kv_head_num != 0)
    return fail(ELLM_ERR_INVALID_ARGUMENT, "attention_head_num %zu is not a multiple of kv_head_num %zu",
                d->attention_head_num, d->kv_head_num);
  if (d->kv_strides[3] != 1)
    return fail(ELLM_ERR_INVALID_ARGUMENT, "kv_strides[3] must be 1 (head dimension contiguous)");
  for (int i = 0; i < 3; ++i)
    if (d->kv_strides[i] == 0 || d->kv_strides[i] % 8 != 0)
      return fail(ELLM_ERR_INVALID_ARGUMENT,
                  "kv_strides[%d] = %zu must be a non-zero multiple of 8 elements", i,
                  d->kv_strides[i]);
  if (d->kv_strides[2] < d->head_size)
    return fail(ELLM_ERR_INVALID_ARGUMENT, "kv_strides[2] = %zu is smaller than head_size",
                d->kv_strides[2]);
  if (d->sequence_capacity == 0 || d->sequence_capacity > 0x7fffffffu)
    return fail(ELLM_ERR_INVALID_ARGUMENT, "sequence_capacity %zu out of range", d->sequence_capacity);
  if (d->sequence_capacity * d->kv_strides[2] > 0x7fffffffu)
    return fail(ELLM_ERR_UNSUPPORTED,
                "a K/V plane spans %zu elements; offsets inside a plane are 32-bit (max 2^31 - 1)",
                d->sequence_capacity * d->kv_strides[2]);
  if (d->max_position_interval == 0 || d->max_position_interval > d->sequence_capacity)
    return fail(ELLM_ERR_INVALID_ARGUMENT,
                "max_position_interval %zu must be in 1..sequence_capacity", d->max_position_interval);
  if (d->batch_size > 65535 || d->attention_head_num > 65535)
    return fail(ELLM_ERR_UNSUPPORTED, "batch_size and attention_head_num are limited to 65535");
  if (!(d->inverse_sqrt_head == d->inverse_sqrt_head))
    return fail(ELLM_ERR_INVALID_ARGUMENT, "inverse_sqrt_head is NaN");
  return ELLM_OK;
}

void ellm::attn_args_from_desc(const ellm_attn_desc& d, ellm::AttnArgs* a) {
  a->q = d.q;
  a->k = d.k;
  a->v = d.v;
  a->out = d.out;
  a->lse = d.lse;
  a->batch_pitch = (uint32_t)d.batch_size;
  a->n_q_heads = (uint32_t)d.attention_head_num;
  a->n_kv_heads = (uint32_t)d.kv_head_num;
  a->group = a->n_q_heads / a->n_kv_heads;
  a->kv_stride_seq = d.kv_strides[0];
  a->kv_stride_head = d.kv_strides[1];
  a->kv_stride_pos = d.kv_strides[2];
  a->scale = d.inverse_sqrt_head;
  a->dtype = d.dtype;
  a->capacity = (uint32_t)d.sequence_capacity;
  a->ws_acc = a->ws_ml = a->ws2_acc = a->ws2_ml = nullptr;
  a->counters = nullptr;
  a->prefill_part_o = a->prefill_part_ml = nullptr;
  a->prefill_part_rows = 0;
  a->n_cu = 0;
  a->positions = nullptr;
}

struct ellm_attn {
  ellm_attn_desc desc;
  int device;
  int n_cu;
  float* ws_acc;
  float* ws_ml;
  float* ws2_acc;
  float* ws2_ml;
  uint32_t* counters;
  ellm::DecodeWorkspace ws;
  // chunk calls with few row blocks on a long cache split the key range: partial rows
  float* part_o;
  float* part_ml;
  size_t part_rows;
};

struct ellm_kv_cache {
  ellm_kv_desc desc;
  int device;
  void* k;
  void* v;
  size_t layer_elems;  // elements per layer
};

static hipError_t free_workspace(ellm_attn* h) {
  hipError_t first = hipSuccess;
  void* ptrs[] = {h->ws_acc, h->ws_ml, h->ws2_acc, h->ws2_ml, h->counters, h->part_o, h->part_ml};
  for (void* p : ptrs) {
    if (!p) continue;
    hipError_t e = hipFree(p);
    if (e != hipSuccess && first == hipSuccess) first = e;
  }
  h->ws_acc = h->ws_ml = h->ws2_acc = h->ws2_ml = h->part_o = h->part_ml = nullptr;
  h->counters = nullptr;
  return first;
}

extern "C" {

const char* ellm_last_error_string(void) { return g_error; }

int ellm_attn_version(void) { return 100; }

int ellm_device_count(void) {
  int n = 0;
  if (hipGetDeviceCount(&n) != hipSuccess) {
    (void)hipGetLastError();
    return 0;
  }
  int usable = 0;
  for (int d = 0; d < n; ++d) {
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, d) == hipSuccess &&
        strncmp(prop.gcnArchName, "gfx950", 6) == 0)
      ++usable;
  }
  return usable;
}

int ellm_attn_create(const ellm_attn_desc* d, ellm_attn** out_handle) {
  if (!d || !out_handle) return fail(ELLM_ERR_INVALID_ARGUMENT, "null descriptor or handle pointer");
  *out_handle = nullptr;
  if (int st = ellm::validate_attn_desc(d)) return st;

  int device = 0, n_cu = 0;
  int st = ellm::current_gfx950_device(&device, &n_cu);
  if (st != ELLM_OK) return st;
  ellm::prepare_static_scratch();

  ellm_attn* h = new (std::nothrow) ellm_attn;
  if (!h) return fail(ELLM_ERR_HIP, "out of host memory");
  h->desc = *d;
  h->device = device;
  h->n_cu = n_cu;
  h->ws = ellm::decode_workspace((uint32_t)d->batch_size, (uint32_t)d->attention_head_num,
                                 (uint32_t)d->kv_head_num, (uint32_t)n_cu);
  h->ws_acc = h->ws_ml = h->ws2_acc = h->ws2_ml = h->part_o = h->part_ml = nullptr;
  h->counters = nullptr;
  h->part_rows = ellm::prefill_workspace_rows((uint32_t)d->max_position_interval, (uint32_t)d->batch_size,
                                              (uint32_t)d->attention_head_num, (uint32_t)n_cu);
  hipError_t e = hipMalloc((void**)&h->ws_acc, h->ws.rows * 128 * sizeof(float));
  if (e == hipSuccess) e = hipMalloc((void**)&h->ws_ml, h->ws.rows * 2 * sizeof(float));
  if (e == hipSuccess) e = hipMalloc((void**)&h->ws2_acc, h->ws.rows2 * 128 * sizeof(float));
  if (e == hipSuccess) e = hipMalloc((void**)&h->ws2_ml, h->ws.rows2 * 2 * sizeof(float));
  // arrival counters of the single-token kernel; they return to zero by themselves
  if (e == hipSuccess) e = hipMalloc((void**)&h->counters, h->ws.counters * sizeof(uint32_t));
  if (e == hipSuccess) e = hipMemset(h->counters, 0, h->ws.counters * sizeof(uint32_t));
  if (e == hipSuccess && h->part_rows) e = hipMalloc((void**)&h->part_o, h->part_rows * 128 * sizeof(float));
  if (e == hipSuccess && h->part_rows) e = hipMalloc((void**)&h->part_ml, h->part_rows * 2 * sizeof(float));
  if (e != hipSuccess) {
    (void)free_workspace(h);
    delete h;
    return fail_hip(e, "hipMalloc(workspace)");
  }
  *out_handle = h;
  return ELLM_OK;
}

int ellm_attn_destroy(ellm_attn* h) {
  if (!h) return ELLM_OK;
  hipError_t e = free_workspace(h);
  delete h;
  if (e != hipSuccess) return fail_hip(e, "hipFree");
  return ELLM_OK;
}

static void fill_args(const ellm_attn* h, ellm::AttnArgs* a) {
  ellm::attn_args_from_desc(h->desc, a);
  a->ws_acc = h->ws_acc;
  a->ws_ml = h->ws_ml;
  a->ws2_acc = h->ws2_acc;
  a->ws2_ml = h->ws2_ml;
  a->counters = h->counters;
  a->prefill_part_o = h->part_o;
  a->prefill_part_ml = h->part_ml;
  a->prefill_part_rows = h->part_rows;
  a->n_cu = (uint32_t)h->n_cu;
}

static int run_decode(ellm_attn* h, ellm::AttnArgs* a, uint32_t max_position, hipStream_t stream) {
  const ellm::DecodePlan plan =
      ellm::decode_plan(max_position + 1, a->batch, a->n_kv_heads, (uint32_t)h->n_cu);
  a->split_len = plan.split_len;
  a->n_split = plan.n_split;
  if (!ellm::decode_plan_fits(h->ws, a->batch, a->n_q_heads, a->n_kv_heads, a->group, a->n_split))
    return fail(ELLM_ERR_OUT_OF_RANGE, "internal: split plan exceeds the workspace");
  hipError_t e = ellm::launch_decode(*a, stream);
  if (e != hipSuccess) return fail_hip(e, "single-token attention launch");
  return ELLM_OK;
}

int ellm_attn_run(ellm_attn* h, size_t position_index, size_t position_interval, size_t batch_size,
                  void* stream) {
  if (!h) return fail(ELLM_ERR_INVALID_ARGUMENT, "null handle");
  if (batch_size == 0 || position_interval == 0) return ELLM_OK;
  if (int st = ellm::check_current_device(h->device)) return st;
  const ellm_attn_desc& d = h->desc;
  if (batch_size > d.batch_size)
    return fail(ELLM_ERR_OUT_OF_RANGE, "batch_size %zu exceeds the capacity %zu", batch_size,
                d.batch_size);
  if (position_interval > d.max_position_interval)
    return fail(ELLM_ERR_OUT_OF_RANGE, "position_interval %zu exceeds max_position_interval %zu",
                position_interval, d.max_position_interval);
  if (position_index >= d.sequence_capacity ||
      position_interval > d.sequence_capacity - position_index)
    return fail(ELLM_ERR_OUT_OF_RANGE,
                "positions [%zu, %zu) do not fit the sequence capacity %zu", position_index,
                position_index + position_interval, d.sequence_capacity);
  ellm::AttnArgs a;
  fill_args(h, &a);
  a.position_index = (uint32_t)position_index;
  a.position_interval = (uint32_t)position_interval;
  a.batch = (uint32_t)batch_size;
  if (position_interval == 1) return run_decode(h, &a, (uint32_t)position_index, (hipStream_t)stream);
  hipError_t e = ellm::launch_prefill(a, (hipStream_t)stream);
  if (e != hipSuccess) return fail_hip(e, "chunk attention launch");
  return ELLM_OK;
}

int ellm_attn_run_ragged(ellm_attn* h, const uint32_t* positions, size_t max_position,
                         size_t batch_size, void* stream) {
  if (!h) return fail(ELLM_ERR_INVALID_ARGUMENT, "null handle");
  if (batch_size == 0) return ELLM_OK;
  if (!positions) return fail(ELLM_ERR_INVALID_ARGUMENT, "null positions");
  if (int st = ellm::check_current_device(h->device)) return st;
  const ellm_attn_desc& d = h->desc;
  if (batch_size > d.batch_size)
    return fail(ELLM_ERR_OUT_OF_RANGE, "batch_size %zu exceeds the capacity %zu", batch_size,
                d.batch_size);
  if (max_position >= d.sequence_capacity)
    return fail(ELLM_ERR_OUT_OF_RANGE, "max_position %zu is not below the sequence capacity %zu",
                max_position, d.sequence_capacity);
  ellm::AttnArgs a;
  fill_args(h, &a);
  a.position_index = (uint32_t)max_position;
  a.position_interval = 1;
  a.batch = (uint32_t)batch_size;
  a.positions = positions;
  return run_decode(h, &a, (uint32_t)max_position, (hipStream_t)stream);
}

/* ---- K/V cache ---------------------------------------------------------- */

int ellm_kv_create(const ellm_kv_desc* d, ellm_kv_cache** out_cache) {
  if (!d || !out_cache) return fail(ELLM_ERR_INVALID_ARGUMENT, "null descriptor or cache pointer");
  *out_cache = nullptr;
  if (d->dtype != ELLM_DTYPE_F16 && d->dtype != ELLM_DTYPE_BF16)
    return fail(ELLM_ERR_INVALID_ARGUMENT, "dtype %d is neither ELLM_DTYPE_F16 nor ELLM_DTYPE_BF16",
                d->dtype);
  if (d->head_size != 128)
    return fail(ELLM_ERR_UNSUPPORTED, "head_size %zu: only 128 is supported", d->head_size);
  if (d->layers == 0 || d->sequences == 0 || d->kv_head_num == 0 || d->capacity == 0)
    return fail(ELLM_ERR_INVALID_ARGUMENT, "layers, sequences, kv_head_num and capacity must be > 0");
  if (d->capacity > 0x7fffffffu || d->sequences > 65535 || d->kv_head_num > 65535)
    return fail(ELLM_ERR_UNSUPPORTED, "capacity / sequences / kv_head_num too large");
  // capacity, sequences and kv_head_num are bounded above; layers is not
  size_t layer_elems = d->sequences * d->kv_head_num;
  size_t bytes = 0;
  if (__builtin_mul_overflow(layer_elems, d->capacity * d->head_size, &layer_elems) ||
      __builtin_mul_overflow(layer_elems, d->layers, &bytes) ||
      __builtin_mul_overflow(bytes, (size_t)2, &bytes))
    return fail(ELLM_ERR_UNSUPPORTED, "the cache's size in bytes does not fit 64 bits");
  int device = 0, n_cu = 0;
  int st = ellm::current_gfx950_device(&device, &n_cu);
  if (st != ELLM_OK) return st;
  ellm::prepare_static_scratch();

  ellm_kv_cache* c = new (std::nothrow) ellm_kv_cache;
  if (!c) return fail(ELLM_ERR_HIP, "out of host memory");
  c->desc = *d;
  c->device = device;
  c->layer_elems = layer_elems;
  c->k = c->v = nullptr;
  hipError_t e = hipMalloc(&c->k, bytes);
  if (e == hipSuccess) e = hipMalloc(&c->v, bytes);
  if (e == hipSuccess) e = hipMemset(c->k, 0, bytes);
  if (e == hipSuccess) e = hipMemset(c->v, 0, bytes);
  if (e != hipSuccess) {
    if (c->k) (void)hipFree(c->k);
    if (c->v) (void)hipFree(c->v);
    delete c;
    return fail_hip(e, "K/V cache allocation");
  }
  *out_cache = c;
  return ELLM_OK;
}

int ellm_kv_destroy(ellm_kv_cache* c) {
  if (!c) return ELLM_OK;
  hipError_t e1 = hipFree(c->k);
  hipError_t e2 = hipFree(c->v);
  delete c;
  if (e1 != hipSuccess) return fail_hip(e1, "hipFree");
  if (e2 != hipSuccess) return fail_hip(e2, "hipFree");
  return ELLM_OK;
}

int ellm_kv_layer(const ellm_kv_cache* c, size_t layer, void** k, void** v, size_t kv_strides[4]) {
  if (!c || !k || !v || !kv_strides) return fail(ELLM_ERR_INVALID_ARGUMENT, "null argument");
  if (layer >= c->desc.layers)
    return fail(ELLM_ERR_OUT_OF_RANGE, "layer %zu of %zu", layer, c->desc.layers);
  *k = (char*)c->k + layer * c->layer_elems * 2;
  *v = (char*)c->v + layer * c->layer_elems * 2;
  kv_strides[0] = c->desc.kv_head_num * c->desc.capacity * c->desc.head_size;
  kv_strides[1] = c->desc.capacity * c->desc.head_size;
  kv_strides[2] = c->desc.head_size;
  kv_strides[3] = 1;
  return ELLM_OK;
}

int ellm_kv_append(ellm_kv_cache* c, size_t layer, size_t position_index, size_t n_tokens,
                   size_t batch_size, const void* k_src, const void* v_src, size_t src_batch_pitch,
                   void* stream) {
  if (!c) return fail(ELLM_ERR_INVALID_ARGUMENT, "null cache");
  if (n_tokens == 0 || batch_size == 0) return ELLM_OK;
  if (!k_src || !v_src) return fail(ELLM_ERR_INVALID_ARGUMENT, "null source");
  if (int st = ellm::check_current_device(c->device)) return st;
  if (!aligned16(k_src) || !aligned16(v_src))
    return fail(ELLM_ERR_INVALID_ARGUMENT, "sources must be 16-byte aligned");
  if (layer >= c->desc.layers)
    return fail(ELLM_ERR_OUT_OF_RANGE, "layer %zu of %zu", layer, c->desc.layers);
  if (batch_size > c->desc.sequences || src_batch_pitch < batch_size)
    return fail(ELLM_ERR_OUT_OF_RANGE, "batch_size %zu exceeds the cache's %zu sequences or the source pitch %zu",
                batch_size, c->desc.sequences, src_batch_pitch);
  if (position_index >= c->desc.capacity || n_tokens > c->desc.capacity - position_index)
    return fail(ELLM_ERR_OUT_OF_RANGE, "positions [%zu, %zu) do not fit the capacity %zu",
                position_index, position_index + n_tokens, c->desc.capacity);
  if (n_tokens > 0xffffffffu / 2 || src_batch_pitch > 65535)
    return fail(ELLM_ERR_UNSUPPORTED, "n_tokens or src_batch_pitch too large");
  void* k = (char*)c->k + layer * c->layer_elems * 2;
  void* v = (char*)c->v + layer * c->layer_elems * 2;
  hipError_t e = ellm::launch_kv_append(k, v, k_src, v_src, (uint32_t)n_tokens, (uint32_t)batch_size,
                                        (uint32_t)src_batch_pitch, (uint32_t)c->desc.kv_head_num,
                                        (uint32_t)c->desc.capacity, (uint32_t)position_index,
                                        (hipStream_t)stream);
  if (e != hipSuccess) return fail_hip(e, "kv append launch");
  return ELLM_OK;
}

int ellm_kv_append_norm_rope(ellm_kv_cache* c, size_t layer, size_t position_index, size_t n_tokens,
                             size_t batch_size, const void* k_src, const void* v_src,
                             size_t src_batch_pitch, const void* rope, size_t rope_positions,
                             float eps, const uint32_t* positions, size_t max_position,
                             void* stream) {
  if (!c) return fail(ELLM_ERR_INVALID_ARGUMENT, "null cache");
  if (n_tokens == 0 || batch_size == 0) return ELLM_OK;
  if (!k_src || !v_src || !rope) return fail(ELLM_ERR_INVALID_ARGUMENT, "null source or rotary table");
  if (int st = ellm::check_current_device(c->device)) return st;
  if (!aligned16(k_src) || !aligned16(v_src) || !aligned16(rope))
    return fail(ELLM_ERR_INVALID_ARGUMENT, "sources and rotary table must be 16-byte aligned");
  if (!(eps >= 0.0f)) return fail(ELLM_ERR_INVALID_ARGUMENT, "eps must be >= 0");
  if (layer >= c->desc.layers)
    return fail(ELLM_ERR_OUT_OF_RANGE, "layer %zu of %zu", layer, c->desc.layers);
  if (batch_size > c->desc.sequences || src_batch_pitch < batch_size)
    return fail(ELLM_ERR_OUT_OF_RANGE, "batch_size %zu exceeds the cache's %zu sequences or the source pitch %zu",
                batch_size, c->desc.sequences, src_batch_pitch);
  // with per-sequence positions the highest start is max_position (entries above it are clamped)
  const size_t first = positions ? max_position : position_index;
  if (first >= c->desc.capacity || n_tokens > c->desc.capacity - first)
    return fail(ELLM_ERR_OUT_OF_RANGE, "positions [%zu, %zu) do not fit the capacity %zu", first,
                first + n_tokens, c->desc.capacity);
  if (first + n_tokens > rope_positions)
    return fail(ELLM_ERR_OUT_OF_RANGE, "positions [%zu, %zu) are beyond the %zu rows of the rotary table",
                first, first + n_tokens, rope_positions);
  if (n_tokens > 0xffffffffu / 2 || src_batch_pitch > 65535)
    return fail(ELLM_ERR_UNSUPPORTED, "n_tokens or src_batch_pitch too large");
  void* k = (char*)c->k + layer * c->layer_elems * 2;
  void* v = (char*)c->v + layer * c->layer_elems * 2;
  hipError_t e = ellm::launch_kv_append_norm_rope(
      k, v, k_src, v_src, rope, positions, (uint32_t)n_tokens, (uint32_t)batch_size,
      (uint32_t)src_batch_pitch, (uint32_t)c->desc.kv_head_num, (uint32_t)c->desc.capacity,
      (uint32_t)position_index, (uint32_t)max_position, eps, c->desc.dtype, (hipStream_t)stream);
  if (e != hipSuccess) return fail_hip(e, "kv append (norm + rope) launch");
  return ELLM_OK;
}

int ellm_schedule_calls(size_t prompt_begin, size_t prompt_end, size_t chunk, size_t generation_end,
                        ellm_call* calls, size_t capacity, size_t* n_calls) {
  if (!n_calls) return fail(ELLM_ERR_INVALID_ARGUMENT, "null n_calls");
  if (chunk == 0) return fail(ELLM_ERR_INVALID_ARGUMENT, "chunk must be positive");
  if (prompt_end < prompt_begin)
    return fail(ELLM_ERR_INVALID_ARGUMENT, "prompt_end %zu before prompt_begin %zu", prompt_end,
                prompt_begin);
  if (capacity && !calls) return fail(ELLM_ERR_INVALID_ARGUMENT, "null calls");
  size_t n = 0;
  auto push = [&](size_t pos, size_t interval) {
    if (n < capacity) calls[n] = ellm_call{pos, interval};
    ++n;
  };
  const size_t prompt = prompt_end - prompt_begin;
  if (prompt) {
    const size_t full = (prompt - 1) / chunk;  // chunks before the last one
    for (size_t i = 0; i < full; ++i) push(prompt_begin + i * chunk, chunk);
    push(prompt_begin + full * chunk, prompt - full * chunk);
  }
  for (size_t pos = prompt_end; pos < generation_end; ++pos) push(pos, 1);
  *n_calls = n;
  if (n > capacity) return fail(ELLM_ERR_OUT_OF_RANGE, "%zu calls, room for %zu", n, capacity);
  return ELLM_OK;
}

struct ellm_graph {
  hipGraph_t graph;
  hipGraphExec_t exec;
};

int ellm_graph_begin(void* stream) {
  if (!stream) return fail(ELLM_ERR_INVALID_ARGUMENT, "the null stream cannot be recorded");
  // relaxed mode: other host threads may keep calling into the runtime meanwhile
  hipError_t e = hipStreamBeginCapture((hipStream_t)stream, hipStreamCaptureModeRelaxed);
  if (e != hipSuccess) return fail_hip(e, "hipStreamBeginCapture");
  return ELLM_OK;
}

int ellm_graph_end(void* stream, ellm_graph** out_graph) {
  if (!stream || !out_graph) return fail(ELLM_ERR_INVALID_ARGUMENT, "null stream or output");
  *out_graph = nullptr;
  hipGraph_t g = nullptr;
  hipError_t e = hipStreamEndCapture((hipStream_t)stream, &g);
  if (e != hipSuccess) return fail_hip(e, "hipStreamEndCapture");
  hipGraphExec_t x = nullptr;
  e = hipGraphInstantiate(&x, g, nullptr, nullptr, 0);
  if (e != hipSuccess) {
    (void)hipGraphDestroy(g);
    return fail_hip(e, "hipGraphInstantiate");
  }
  ellm_graph* h = new (std::nothrow) ellm_graph{g, x};
  if (!h) {
    (void)hipGraphExecDestroy(x);
    (void)hipGraphDestroy(g);
    return fail(ELLM_ERR_HIP, "out of host memory");
  }
  *out_graph = h;
  return ELLM_OK;
}

int ellm_graph_launch(ellm_graph* graph, void* stream) {
  if (!graph) return fail(ELLM_ERR_INVALID_ARGUMENT, "null graph");
  hipError_t e = hipGraphLaunch(graph->exec, (hipStream_t)stream);
  if (e != hipSuccess) return fail_hip(e, "hipGraphLaunch");
  return ELLM_OK;
}

int ellm_graph_destroy(ellm_graph* graph) {
  if (!graph) return ELLM_OK;
  hipError_t e1 = hipGraphExecDestroy(graph->exec);
  hipError_t e2 = hipGraphDestroy(graph->graph);
  delete graph;
  if (e1 != hipSuccess) return fail_hip(e1, "hipGraphExecDestroy");
  if (e2 != hipSuccess) return fail_hip(e2, "hipGraphDestroy");
  return ELLM_OK;
}

int ellm_positions_advance(uint32_t* positions, size_t batch_size, uint32_t by, void* stream) {
  if (batch_size == 0) return ELLM_OK;
  if (!positions) return fail(ELLM_ERR_INVALID_ARGUMENT, "null positions");
  if (batch_size > 0xffffffffu) return fail(ELLM_ERR_UNSUPPORTED, "batch_size too large");
  hipError_t e =
      ellm::launch_positions_advance(positions, (uint32_t)batch_size, by, (hipStream_t)stream);
  if (e != hipSuccess) return fail_hip(e, "positions advance launch");
  return ELLM_OK;
}

}  // extern "C"
