// C ABI of the attention path (declared in include/ellm_attn.h): argument
// validation, the operator handle, the K/V cache object, error reporting.
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <new>
#include <vector>

#include "../../include/ellm_attn.h"
#include "handles.hpp"
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

bool ellm::attn_is_general(const ellm_attn_desc& d) { return d.head_size != 128 || d.dtype == ELLM_DTYPE_F32; }

int ellm::validate_attn_desc(const ellm_attn_desc* d) {
  if (!d) return fail(ELLM_ERR_INVALID_ARGUMENT, "null descriptor");
  if (!d->q || !d->k || !d->v || !d->out)
    return fail(ELLM_ERR_INVALID_ARGUMENT, "q, k, v and out must be non-null device pointers");
  if (!aligned16(d->q) || !aligned16(d->k) || !aligned16(d->v) || !aligned16(d->out))
    return fail(ELLM_ERR_INVALID_ARGUMENT, "q, k, v and out must be 16-byte aligned");
  if (d->dtype != ELLM_DTYPE_F16 && d->dtype != ELLM_DTYPE_BF16 && d->dtype != ELLM_DTYPE_F32)
    return fail(ELLM_ERR_INVALID_ARGUMENT, "dtype %d is none of ELLM_DTYPE_F16, ELLM_DTYPE_BF16, ELLM_DTYPE_F32",
                d->dtype);
  if (d->head_size == 0 || d->head_size > 256)
    return fail(ELLM_ERR_UNSUPPORTED, "head_size %zu: 1 to 256 are supported", d->head_size);
  const bool general = ellm::attn_is_general(*d);
  if (d->batch_size == 0 || d->attention_head_num == 0 || d->kv_head_num == 0)
    return fail(ELLM_ERR_INVALID_ARGUMENT, "batch_size, attention_head_num, kv_head_num must be > 0");
  if (d->attention_head_num % d->kv_head_num != 0)
    return fail(ELLM_ERR_INVALID_ARGUMENT, "attention_head_num %zu is not a multiple of kv_head_num %zu",
                d->attention_head_num, d->kv_head_num);
  if (d->kv_strides[3] != 1)
    return fail(ELLM_ERR_INVALID_ARGUMENT, "kv_strides[3] must be 1 (head dimension contiguous)");
  for (int i = 0; i < 3; ++i)
    if (d->kv_strides[i] == 0 || (!general && d->kv_strides[i] % 8 != 0))
      return fail(ELLM_ERR_INVALID_ARGUMENT,
                  "kv_strides[%d] = %zu must be a non-zero multiple of 8 elements (non-zero for head sizes "
                  "other than 128 and for binary32)", i, d->kv_strides[i]);
  if (d->kv_strides[2] < d->head_size)
    return fail(ELLM_ERR_INVALID_ARGUMENT, "kv_strides[2] = %zu is smaller than head_size",
                d->kv_strides[2]);
  if (d->sequence_capacity == 0 || d->sequence_capacity > 0x7fffffffu)
    return fail(ELLM_ERR_INVALID_ARGUMENT, "sequence_capacity %zu out of range", d->sequence_capacity);
  // offsets inside a plane are 64-bit; a tile of 64 rows is addressed with 32-bit byte offsets
  if (d->kv_strides[2] > ((size_t)1 << 24))
    return fail(ELLM_ERR_UNSUPPORTED,
                "kv_strides[2] = %zu elements: rows of a K/V plane may be at most 2^24 elements apart",
                d->kv_strides[2]);
  size_t span = 0;
  if (__builtin_mul_overflow(d->sequence_capacity, d->kv_strides[2], &span) || span > ((size_t)1 << 46))
    return fail(ELLM_ERR_UNSUPPORTED, "a K/V plane spans more than 2^46 elements");
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
  a->seq_offsets = nullptr;
  a->seq_caps = nullptr;
  a->pending = ellm::PendingRows{};
}

struct ellm_kv_cache {
  ellm_kv_desc desc;   // capacity = the largest per-sequence capacity
  int device;
  void* k;
  void* v;
  size_t layer_elems;  // elements per layer
  // plane of (sequence s, head h) = layer base + offset(s) + h x stride_head.  One capacity for
  // all: [sequence][kv_head][position][128], offset(s) = s x stride_seq, no tables.  Per-sequence
  // capacities: [kv_head][sequence: its positions][128], offset(s) = 128 x (positions of the
  // sequences before s), kept in a device table (and capacities beside it).
  size_t stride_seq, stride_head;
  bool ragged;
  std::vector<size_t> caps_host;      // [sequences]
  std::vector<size_t> offsets_host;   // [sequences], elements
  size_t* seq_offsets_dev;            // ragged only
  uint32_t* seq_caps_dev;             // ragged only
  ellm::KvLayout layout(size_t first_sequence = 0) const {
    ellm::KvLayout l;
    l.stride_seq = stride_seq;
    l.stride_head = stride_head;
    l.seq_offsets = ragged ? seq_offsets_dev + first_sequence : nullptr;
    l.seq_caps = ragged ? seq_caps_dev + first_sequence : nullptr;
    return l;
  }
  // the smallest / largest capacity among sequences [0, n)
  size_t min_cap(size_t n) const {
    size_t m = caps_host[0];
    for (size_t i = 1; i < n; ++i) m = caps_host[i] < m ? caps_host[i] : m;
    return m;
  }
  size_t max_cap(size_t n) const {
    size_t m = caps_host[0];
    for (size_t i = 1; i < n; ++i) m = caps_host[i] > m ? caps_host[i] : m;
    return m;
  }
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

static int attn_create(const ellm_attn_desc* d, const ellm_kv_seq_table* table, ellm_attn** out_handle) {
  if (!d || !out_handle) return fail(ELLM_ERR_INVALID_ARGUMENT, "null descriptor or handle pointer");
  *out_handle = nullptr;
  ellm_attn_desc local;
  if (table) {
    if (!table->seq_offsets || !table->seq_capacity || !table->seq_capacity_host)
      return fail(ELLM_ERR_INVALID_ARGUMENT, "the sequence table has a null member");
    if (d->batch_size == 0 || d->batch_size > table->sequences)
      return fail(ELLM_ERR_OUT_OF_RANGE, "batch_size %zu, the sequence table has %zu entries", d->batch_size,
                  table->sequences);
    // sequence_capacity is the largest capacity among the operator's sequences; kv_strides[0]
    // has no meaning (the table gives every sequence's offset) and only has to pass the checks
    local = *d;
    size_t cap = 0;
    for (size_t i = 0; i < d->batch_size; ++i) {
      if (table->seq_capacity_host[i] == 0)
        return fail(ELLM_ERR_INVALID_ARGUMENT, "sequence %zu of the table has capacity 0", i);
      cap = table->seq_capacity_host[i] > cap ? table->seq_capacity_host[i] : cap;
    }
    local.sequence_capacity = cap;
    if (local.kv_strides[0] == 0) local.kv_strides[0] = 8;
    d = &local;
  }
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
  h->seq_offsets = nullptr;
  h->seq_caps = nullptr;
  if (table) {
    h->seq_offsets = table->seq_offsets;
    h->seq_caps = table->seq_capacity;
    h->caps_host.assign(table->seq_capacity_host, table->seq_capacity_host + d->batch_size);
  }
  h->ws = ellm::decode_workspace((uint32_t)d->batch_size, (uint32_t)d->attention_head_num,
                                 (uint32_t)d->kv_head_num, (uint32_t)n_cu);
  h->ws_acc = h->ws_ml = h->ws2_acc = h->ws2_ml = h->part_o = h->part_ml = nullptr;
  h->counters = nullptr;
  h->part_rows = ellm::prefill_workspace_rows((uint32_t)d->max_position_interval, (uint32_t)d->batch_size,
                                              (uint32_t)d->attention_head_num, (uint32_t)n_cu);
  h->general = ellm::attn_is_general(*d);
  if (h->general) {   // the kernel for other head sizes and binary32 keeps nothing between workgroups
    h->ws = ellm::DecodeWorkspace{0, 0, 0};
    h->part_rows = 0;
    *out_handle = h;
    return ELLM_OK;
  }
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

int ellm_attn_create(const ellm_attn_desc* d, ellm_attn** out_handle) {
  return attn_create(d, nullptr, out_handle);
}

int ellm_attn_create_ragged(const ellm_attn_desc* d, const ellm_kv_seq_table* table,
                            ellm_attn** out_handle) {
  if (!table) return fail(ELLM_ERR_INVALID_ARGUMENT, "null sequence table");
  return attn_create(d, table, out_handle);
}

int ellm_attn_reset(ellm_attn* h, void* stream) {
  if (!h) return fail(ELLM_ERR_INVALID_ARGUMENT, "null handle");
  if (int st = ellm::check_current_device(h->device)) return st;
  if (h->general) return ELLM_OK;   // no counters
  const hipError_t e = ellm::launch_fill_u32(h->counters, h->ws.counters, 0u, (hipStream_t)stream);
  if (e != hipSuccess) return fail_hip(e, "counter reset launch");
  return ELLM_OK;
}

int ellm_attn_destroy(ellm_attn* h) {
  if (!h) return ELLM_OK;
  hipError_t e = free_workspace(h);
  delete h;
  if (e != hipSuccess) return fail_hip(e, "hipFree");
  return ELLM_OK;
}

}  // extern "C"

void ellm::attn_fill_args(const ellm_attn* h, ellm::AttnArgs* a) {
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
  a->seq_offsets = h->seq_offsets;
  a->seq_caps = h->seq_caps;
}

// sequences of different lengths: equal shares of all keys; two workgroups per compute unit are
// launched, and the kernel lets one or two per unit take part (it knows the lengths)
static bool takes_balanced(const ellm_attn* h, size_t batch, size_t max_position, uint32_t* wgs) {
  *wgs = 2 * (uint32_t)h->n_cu;
  const ellm_attn_desc& d = h->desc;
  return ellm::decode_balanced_takes(h->ws, (uint32_t)batch, (uint32_t)d.kv_head_num,
                                     (uint32_t)(d.attention_head_num / d.kv_head_num),
                                     (uint32_t)max_position + 1, *wgs);
}

int ellm::attn_run_single_token(ellm_attn* h, ellm::AttnArgs* a, uint32_t max_position, hipStream_t stream) {
  if (h->general) {
    const hipError_t e = ellm::launch_attn_general(*a, (uint32_t)h->desc.head_size, stream);
    if (e != hipSuccess) return fail_hip(e, "attention launch (general head size)");
    return ELLM_OK;
  }
  uint32_t wgs = 0;
  if (a->positions && takes_balanced(h, a->batch, max_position, &wgs)) {
    const hipError_t e = ellm::launch_decode_balanced(*a, wgs, stream);
    if (e != hipSuccess) return fail_hip(e, "single-token attention launch");
    return ELLM_OK;
  }
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

extern "C" {

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
  for (size_t i = 0; i < batch_size && i < h->caps_host.size(); ++i)
    if (position_index + position_interval > h->caps_host[i])
      return fail(ELLM_ERR_OUT_OF_RANGE, "positions [%zu, %zu) do not fit sequence %zu, whose capacity is %zu",
                  position_index, position_index + position_interval, i, h->caps_host[i]);
  ellm::AttnArgs a;
  ellm::attn_fill_args(h, &a);
  a.position_index = (uint32_t)position_index;
  a.position_interval = (uint32_t)position_interval;
  a.batch = (uint32_t)batch_size;
  if (position_interval == 1) return ellm::attn_run_single_token(h, &a, (uint32_t)position_index, (hipStream_t)stream);
  hipError_t e = h->general ? ellm::launch_attn_general(a, (uint32_t)d.head_size, (hipStream_t)stream)
                            : ellm::launch_prefill(a, (hipStream_t)stream);
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
  ellm::attn_fill_args(h, &a);
  a.position_index = (uint32_t)max_position;
  a.position_interval = 1;
  a.batch = (uint32_t)batch_size;
  a.positions = positions;
  return ellm::attn_run_single_token(h, &a, (uint32_t)max_position, (hipStream_t)stream);
}

int ellm_attn_ragged_path(const ellm_attn* h, size_t max_position, size_t batch_size) {
  if (!h) return -fail(ELLM_ERR_INVALID_ARGUMENT, "null handle");
  if (batch_size == 0 || batch_size > h->desc.batch_size || max_position >= h->desc.sequence_capacity)
    return -fail(ELLM_ERR_OUT_OF_RANGE, "batch_size %zu / max_position %zu outside the handle's %zu / %zu",
                 batch_size, max_position, h->desc.batch_size, h->desc.sequence_capacity);
  if (h->general) return 0;
  uint32_t wgs = 0;
  return takes_balanced(h, batch_size, max_position, &wgs) ? 1 : 0;
}

/* ---- K/V cache ---------------------------------------------------------- */

// Shared by the two create functions: caps = positions per plane of every sequence;
// uniform -> [sequence][kv_head][position][128] with one capacity, else
// [kv_head][sequence: its own positions][128] with offset / capacity tables on the device.
static int kv_create(size_t layers, size_t kv_head_num, size_t head_size, int dtype,
                     const std::vector<size_t>& caps, bool ragged, ellm_kv_cache** out_cache) {
  if (dtype != ELLM_DTYPE_F16 && dtype != ELLM_DTYPE_BF16)
    return fail(ELLM_ERR_INVALID_ARGUMENT, "dtype %d is neither ELLM_DTYPE_F16 nor ELLM_DTYPE_BF16", dtype);
  if (head_size != 128)
    return fail(ELLM_ERR_UNSUPPORTED, "head_size %zu: only 128 is supported", head_size);
  const size_t sequences = caps.size();
  if (layers == 0 || sequences == 0 || kv_head_num == 0)
    return fail(ELLM_ERR_INVALID_ARGUMENT, "layers, sequences, kv_head_num and capacity must be > 0");
  if (sequences > 65535 || kv_head_num > 65535)
    return fail(ELLM_ERR_UNSUPPORTED, "capacity / sequences / kv_head_num too large");
  size_t total = 0, largest = 0;   // positions of all sequences of one head
  for (size_t cap : caps) {
    if (cap == 0) return fail(ELLM_ERR_INVALID_ARGUMENT, "layers, sequences, kv_head_num and capacity must be > 0");
    if (cap > 0x7fffffffu / 128) return fail(ELLM_ERR_UNSUPPORTED, "capacity / sequences / kv_head_num too large");
    total += cap;   // at most 65535 x 2^24
    largest = cap > largest ? cap : largest;
  }
  // sequences, capacities and kv_head_num are bounded above; layers is not
  size_t layer_elems = total * head_size;
  size_t bytes = 0;
  if (__builtin_mul_overflow(layer_elems, kv_head_num, &layer_elems) ||
      __builtin_mul_overflow(layer_elems, layers, &bytes) ||
      __builtin_mul_overflow(bytes, (size_t)2, &bytes))
    return fail(ELLM_ERR_UNSUPPORTED, "the cache's size in bytes does not fit 64 bits");
  int device = 0, n_cu = 0;
  int st = ellm::current_gfx950_device(&device, &n_cu);
  if (st != ELLM_OK) return st;
  ellm::prepare_static_scratch();

  ellm_kv_cache* c = new (std::nothrow) ellm_kv_cache;
  if (!c) return fail(ELLM_ERR_HIP, "out of host memory");
  c->desc = ellm_kv_desc{layers, sequences, kv_head_num, head_size, largest, dtype};
  c->device = device;
  c->layer_elems = layer_elems;
  c->ragged = ragged;
  c->caps_host = caps;
  c->offsets_host.resize(sequences);
  c->k = c->v = nullptr;
  c->seq_offsets_dev = nullptr;
  c->seq_caps_dev = nullptr;
  if (ragged) {
    c->stride_seq = 0;
    c->stride_head = total * head_size;
    size_t at = 0;
    for (size_t i = 0; i < sequences; ++i) {
      c->offsets_host[i] = at * head_size;
      at += caps[i];
    }
  } else {
    c->stride_seq = kv_head_num * largest * head_size;
    c->stride_head = largest * head_size;
    for (size_t i = 0; i < sequences; ++i) c->offsets_host[i] = i * c->stride_seq;
  }
  hipError_t e = hipMalloc(&c->k, bytes);
  if (e == hipSuccess) e = hipMalloc(&c->v, bytes);
  if (e == hipSuccess) e = hipMemset(c->k, 0, bytes);
  if (e == hipSuccess) e = hipMemset(c->v, 0, bytes);
  if (e == hipSuccess && ragged) {
    std::vector<uint32_t> caps32(caps.begin(), caps.end());
    e = hipMalloc((void**)&c->seq_offsets_dev, sequences * sizeof(size_t));
    if (e == hipSuccess) e = hipMalloc((void**)&c->seq_caps_dev, sequences * sizeof(uint32_t));
    if (e == hipSuccess)
      e = hipMemcpy(c->seq_offsets_dev, c->offsets_host.data(), sequences * sizeof(size_t), hipMemcpyHostToDevice);
    if (e == hipSuccess)
      e = hipMemcpy(c->seq_caps_dev, caps32.data(), sequences * sizeof(uint32_t), hipMemcpyHostToDevice);
  }
  if (e != hipSuccess) {
    if (c->k) (void)hipFree(c->k);
    if (c->v) (void)hipFree(c->v);
    if (c->seq_offsets_dev) (void)hipFree(c->seq_offsets_dev);
    if (c->seq_caps_dev) (void)hipFree(c->seq_caps_dev);
    delete c;
    return fail_hip(e, "K/V cache allocation");
  }
  *out_cache = c;
  return ELLM_OK;
}

int ellm_kv_create(const ellm_kv_desc* d, ellm_kv_cache** out_cache) {
  if (!d || !out_cache) return fail(ELLM_ERR_INVALID_ARGUMENT, "null descriptor or cache pointer");
  *out_cache = nullptr;
  if (d->sequences > 65535) return fail(ELLM_ERR_UNSUPPORTED, "capacity / sequences / kv_head_num too large");
  if (d->capacity > 0x7fffffffu) return fail(ELLM_ERR_UNSUPPORTED, "capacity / sequences / kv_head_num too large");
  // (a size that cannot be allocated must be refused before the per-sequence vectors are built)
  size_t probe = 0;
  if (__builtin_mul_overflow(d->sequences * (d->kv_head_num > 65535 ? 65535 : d->kv_head_num),
                             d->capacity * 128, &probe) ||
      __builtin_mul_overflow(probe, d->layers, &probe) || __builtin_mul_overflow(probe, (size_t)2, &probe))
    return fail(ELLM_ERR_UNSUPPORTED, "the cache's size in bytes does not fit 64 bits");
  if (d->head_size != 128)
    return fail(ELLM_ERR_UNSUPPORTED, "head_size %zu: only 128 is supported", d->head_size);
  const std::vector<size_t> caps(d->sequences, d->capacity);
  return kv_create(d->layers, d->kv_head_num, d->head_size, d->dtype, caps, false, out_cache);
}

int ellm_kv_create_ragged(const ellm_kv_ragged_desc* d, ellm_kv_cache** out_cache) {
  if (!d || !out_cache) return fail(ELLM_ERR_INVALID_ARGUMENT, "null descriptor or cache pointer");
  *out_cache = nullptr;
  if (!d->capacities) return fail(ELLM_ERR_INVALID_ARGUMENT, "null capacities");
  if (d->sequences == 0 || d->sequences > 65535)
    return fail(d->sequences ? ELLM_ERR_UNSUPPORTED : ELLM_ERR_INVALID_ARGUMENT, "sequences %zu out of range", d->sequences);
  const std::vector<size_t> caps(d->capacities, d->capacities + d->sequences);
  return kv_create(d->layers, d->kv_head_num, d->head_size, d->dtype, caps, true, out_cache);
}

int ellm_kv_destroy(ellm_kv_cache* c) {
  if (!c) return ELLM_OK;
  hipError_t e1 = hipFree(c->k);
  hipError_t e2 = hipFree(c->v);
  if (c->seq_offsets_dev) (void)hipFree(c->seq_offsets_dev);
  if (c->seq_caps_dev) (void)hipFree(c->seq_caps_dev);
  delete c;
  if (e1 != hipSuccess) return fail_hip(e1, "hipFree");
  if (e2 != hipSuccess) return fail_hip(e2, "hipFree");
  return ELLM_OK;
}

int ellm_kv_layer(const ellm_kv_cache* c, size_t layer, void** k, void** v, size_t kv_strides[4]) {
  if (!c || !k || !v || !kv_strides) return fail(ELLM_ERR_INVALID_ARGUMENT, "null argument");
  if (c->ragged)
    return fail(ELLM_ERR_INVALID_ARGUMENT,
                "this cache has per-sequence capacities: no single sequence stride exists, use ellm_kv_layer_ragged");
  if (layer >= c->desc.layers)
    return fail(ELLM_ERR_OUT_OF_RANGE, "layer %zu of %zu", layer, c->desc.layers);
  *k = (char*)c->k + layer * c->layer_elems * 2;
  *v = (char*)c->v + layer * c->layer_elems * 2;
  kv_strides[0] = c->stride_seq;
  kv_strides[1] = c->stride_head;
  kv_strides[2] = c->desc.head_size;
  kv_strides[3] = 1;
  return ELLM_OK;
}

int ellm_kv_layer_ragged(const ellm_kv_cache* c, size_t layer, size_t first_sequence, void** k, void** v,
                         size_t kv_strides[4], ellm_kv_seq_table* table) {
  if (!c || !k || !v || !kv_strides || !table) return fail(ELLM_ERR_INVALID_ARGUMENT, "null argument");
  if (!c->ragged)
    return fail(ELLM_ERR_INVALID_ARGUMENT, "this cache has one capacity for every sequence: use ellm_kv_layer");
  if (layer >= c->desc.layers)
    return fail(ELLM_ERR_OUT_OF_RANGE, "layer %zu of %zu", layer, c->desc.layers);
  if (first_sequence >= c->desc.sequences)
    return fail(ELLM_ERR_OUT_OF_RANGE, "first_sequence %zu of %zu", first_sequence, c->desc.sequences);
  *k = (char*)c->k + layer * c->layer_elems * 2;
  *v = (char*)c->v + layer * c->layer_elems * 2;
  kv_strides[0] = c->layer_elems;   // not used with a table (every sequence has its own offset)
  kv_strides[1] = c->stride_head;
  kv_strides[2] = c->desc.head_size;
  kv_strides[3] = 1;
  table->seq_offsets = c->seq_offsets_dev + first_sequence;
  table->seq_capacity = c->seq_caps_dev + first_sequence;
  table->seq_capacity_host = c->caps_host.data() + first_sequence;
  table->sequences = c->desc.sequences - first_sequence;
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
  const size_t room = c->min_cap(batch_size);   // the shortest of the sequences written
  if (position_index >= room || n_tokens > room - position_index)
    return fail(ELLM_ERR_OUT_OF_RANGE, "positions [%zu, %zu) do not fit the capacity %zu",
                position_index, position_index + n_tokens, room);
  if (n_tokens > 0xffffffffu / 2 || src_batch_pitch > 65535)
    return fail(ELLM_ERR_UNSUPPORTED, "n_tokens or src_batch_pitch too large");
  void* k = (char*)c->k + layer * c->layer_elems * 2;
  void* v = (char*)c->v + layer * c->layer_elems * 2;
  hipError_t e = ellm::launch_kv_append(k, v, k_src, v_src, (uint32_t)n_tokens, (uint32_t)batch_size,
                                        (uint32_t)src_batch_pitch, (uint32_t)c->desc.kv_head_num,
                                        c->layout(), (uint32_t)position_index, (hipStream_t)stream);
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
  // (a cache with per-sequence capacities also bounds each sequence's rows on the device)
  const size_t first = positions ? max_position : position_index;
  const size_t room = positions ? c->max_cap(batch_size) : c->min_cap(batch_size);
  if (first >= room || n_tokens > room - first)
    return fail(ELLM_ERR_OUT_OF_RANGE, "positions [%zu, %zu) do not fit the capacity %zu", first,
                first + n_tokens, room);
  if (first + n_tokens > rope_positions)
    return fail(ELLM_ERR_OUT_OF_RANGE, "positions [%zu, %zu) are beyond the %zu rows of the rotary table",
                first, first + n_tokens, rope_positions);
  if (n_tokens > 0xffffffffu / 2 || src_batch_pitch > 65535)
    return fail(ELLM_ERR_UNSUPPORTED, "n_tokens or src_batch_pitch too large");
  void* k = (char*)c->k + layer * c->layer_elems * 2;
  void* v = (char*)c->v + layer * c->layer_elems * 2;
  hipError_t e = ellm::launch_kv_append_norm_rope(
      k, v, k_src, v_src, rope, positions, (uint32_t)n_tokens, (uint32_t)batch_size,
      (uint32_t)src_batch_pitch, (uint32_t)c->desc.kv_head_num, c->layout(),
      (uint32_t)position_index, (uint32_t)max_position, eps, c->desc.dtype, (hipStream_t)stream);
  if (e != hipSuccess) return fail_hip(e, "kv append (norm + rope) launch");
  return ELLM_OK;
}

// Why an attention operator cannot take a layer of a cache as the destination of its own new rows
// (null: it can).
static const char* append_mismatch(const ellm_kv_cache* c, size_t layer, const ellm_attn* a) {
  const ellm_attn_desc& d = a->desc;
  if (a->general) return "the attention operator has a head size other than 128 or binary32 storage";
  if (c->device != a->device) return "the cache and the operator were created on different devices";
  if (d.dtype != c->desc.dtype) return "the cache and the operator differ in dtype";
  if (d.kv_head_num != c->desc.kv_head_num) return "the cache and the operator differ in kv_head_num";
  const void* k = (const char*)c->k + layer * c->layer_elems * 2;
  const void* v = (const char*)c->v + layer * c->layer_elems * 2;
  if (d.k != k || d.v != v) return "the operator's k / v are not this layer of the cache";
  if (d.kv_strides[1] != c->stride_head || d.kv_strides[2] != 128 || d.kv_strides[3] != 1)
    return "the operator's kv_strides are not the cache's";
  if (c->ragged) {
    if (a->seq_offsets != c->seq_offsets_dev || a->seq_caps != c->seq_caps_dev)
      return "the operator was not created with this cache's sequence table (from its first sequence)";
  } else if (a->seq_offsets || d.kv_strides[0] != c->stride_seq) {
    return "the operator's kv_strides are not the cache's";
  }
  return nullptr;
}

static int kv_append_attn(ellm_kv_cache* c, size_t layer, ellm_attn* a, const void* k_src, const void* v_src,
                          const void* rope, size_t rope_positions, float eps, size_t position_index,
                          const uint32_t* positions, size_t max_position, size_t batch_size, void* stream) {
  if (!c || !a) return fail(ELLM_ERR_INVALID_ARGUMENT, "null cache or attention handle");
  if (batch_size == 0) return ELLM_OK;
  if (!k_src || !v_src || !rope) return fail(ELLM_ERR_INVALID_ARGUMENT, "null source or rotary table");
  if (int st = ellm::check_current_device(c->device)) return st;
  if (!aligned16(k_src) || !aligned16(v_src) || !aligned16(rope))
    return fail(ELLM_ERR_INVALID_ARGUMENT, "sources and rotary table must be 16-byte aligned");
  if (!(eps >= 0.0f)) return fail(ELLM_ERR_INVALID_ARGUMENT, "eps must be >= 0");
  if (layer >= c->desc.layers) return fail(ELLM_ERR_OUT_OF_RANGE, "layer %zu of %zu", layer, c->desc.layers);
  if (const char* why = append_mismatch(c, layer, a)) return fail(ELLM_ERR_INVALID_ARGUMENT, "%s", why);
  if (batch_size > c->desc.sequences || batch_size > a->desc.batch_size)
    return fail(ELLM_ERR_OUT_OF_RANGE, "batch_size %zu exceeds the cache's %zu sequences or the operator's %zu",
                batch_size, c->desc.sequences, a->desc.batch_size);
  // the range checks of ellm_kv_append_norm_rope (one token) and of ellm_attn_run / _run_ragged
  const size_t first = positions ? max_position : position_index;
  const size_t room = positions ? c->max_cap(batch_size) : c->min_cap(batch_size);
  if (first >= room) return fail(ELLM_ERR_OUT_OF_RANGE, "position %zu does not fit the capacity %zu", first, room);
  if (first >= rope_positions)
    return fail(ELLM_ERR_OUT_OF_RANGE, "position %zu is beyond the %zu rows of the rotary table", first, rope_positions);
  if (first >= a->desc.sequence_capacity)
    return fail(ELLM_ERR_OUT_OF_RANGE, "position %zu is not below the operator's sequence capacity %zu", first,
                a->desc.sequence_capacity);
  ellm::AttnArgs args;
  ellm::attn_fill_args(a, &args);
  args.position_index = (uint32_t)first;
  args.position_interval = 1;
  args.batch = (uint32_t)batch_size;
  args.positions = positions;
  args.pending.k_rows = k_src;
  args.pending.v_rows = v_src;
  args.pending.rope = rope;
  args.pending.rope_pos_stride = 128;
  args.pending.rope_head_stride = 0;
  args.pending.eps = eps;
  return ellm::attn_run_single_token(a, &args, (uint32_t)first, (hipStream_t)stream);
}

int ellm_kv_append_attn_run(ellm_kv_cache* cache, size_t layer, ellm_attn* attn, size_t position_index,
                            size_t batch_size, const void* k_src, const void* v_src, const void* rope,
                            size_t rope_positions, float eps, void* stream) {
  return kv_append_attn(cache, layer, attn, k_src, v_src, rope, rope_positions, eps, position_index, nullptr, 0,
                        batch_size, stream);
}

int ellm_kv_append_attn_run_ragged(ellm_kv_cache* cache, size_t layer, ellm_attn* attn, const uint32_t* positions,
                                   size_t max_position, size_t batch_size, const void* k_src, const void* v_src,
                                   const void* rope, size_t rope_positions, float eps, void* stream) {
  if (!positions) return fail(ELLM_ERR_INVALID_ARGUMENT, "positions must be a device array");
  return kv_append_attn(cache, layer, attn, k_src, v_src, rope, rope_positions, eps, 0, positions, max_position,
                        batch_size, stream);
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

struct ellm_side_stream {
  int device;
  hipStream_t stream;
  hipEvent_t forked;   // recorded on the caller's stream, awaited by the side stream
  hipEvent_t joined;   // recorded on the side stream, awaited by the caller's stream
};

int ellm_side_stream_create(ellm_side_stream** out) {
  if (!out) return fail(ELLM_ERR_INVALID_ARGUMENT, "null output");
  *out = nullptr;
  int device = 0, n_cu = 0;
  if (int st = ellm::current_gfx950_device(&device, &n_cu)) return st;
  ellm_side_stream* s = new (std::nothrow) ellm_side_stream{device, nullptr, nullptr, nullptr};
  if (!s) return fail(ELLM_ERR_HIP, "out of host memory");
  // (default priority, as every stream that shares the device with the caller's)
  hipError_t e = hipStreamCreateWithFlags(&s->stream, hipStreamNonBlocking);
  if (e == hipSuccess) e = hipEventCreateWithFlags(&s->forked, hipEventDisableTiming);
  if (e == hipSuccess) e = hipEventCreateWithFlags(&s->joined, hipEventDisableTiming);
  if (e != hipSuccess) {
    (void)ellm_side_stream_destroy(s);
    return fail_hip(e, "side stream");
  }
  *out = s;
  return ELLM_OK;
}

void* ellm_side_stream_get(ellm_side_stream* s) { return s ? (void*)s->stream : nullptr; }

int ellm_side_stream_fork(ellm_side_stream* s, void* stream) {
  if (!s) return fail(ELLM_ERR_INVALID_ARGUMENT, "null side stream");
  if (int st = ellm::check_current_device(s->device)) return st;
  hipError_t e = hipEventRecord(s->forked, (hipStream_t)stream);
  if (e == hipSuccess) e = hipStreamWaitEvent(s->stream, s->forked, 0);
  if (e != hipSuccess) return fail_hip(e, "side stream fork");
  return ELLM_OK;
}

int ellm_side_stream_join(ellm_side_stream* s, void* stream) {
  if (!s) return fail(ELLM_ERR_INVALID_ARGUMENT, "null side stream");
  if (int st = ellm::check_current_device(s->device)) return st;
  hipError_t e = hipEventRecord(s->joined, s->stream);
  if (e == hipSuccess) e = hipStreamWaitEvent((hipStream_t)stream, s->joined, 0);
  if (e != hipSuccess) return fail_hip(e, "side stream join");
  return ELLM_OK;
}

int ellm_side_stream_destroy(ellm_side_stream* s) {
  if (!s) return ELLM_OK;
  hipError_t first = hipSuccess;
  auto note = [&](hipError_t e) {
    if (e != hipSuccess && first == hipSuccess) first = e;
  };
  if (s->stream) note(hipStreamSynchronize(s->stream));
  if (s->forked) note(hipEventDestroy(s->forked));
  if (s->joined) note(hipEventDestroy(s->joined));
  if (s->stream) note(hipStreamDestroy(s->stream));
  delete s;
  if (first != hipSuccess) return fail_hip(first, "side stream destroy");
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
