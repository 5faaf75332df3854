// C ABI of the projections either side of attention (declared in
// include/ellm_attn.h): validation and handles for ellm_matmul3_* and
// ellm_matmul_add_*.  A handle owns the workspace of the few-rows kernel only.
#include <hip/hip_runtime.h>

#include <cmath>
#include <new>
#include <vector>

#include "../../include/ellm_attn.h"
#include "handles.hpp"
#include "kernels.hpp"

namespace {
bool aligned16(const void* p) { return ((uintptr_t)p & 15u) == 0; }
constexpr size_t kMaxK = 1u << 16;
}  // namespace

struct ellm_matmul_add {
  ellm_matmul_add_desc d;
  int device;
  float* ws;
  uint32_t* counters;
};

namespace {
// Partial sums and arrival counters of the few-rows kernel; left null (the tile kernel then
// runs every call) when they would take more than 64 MiB.
int alloc_small_workspace(uint32_t heads, uint32_t K, int* device, float** ws, uint32_t** counters) {
  *ws = nullptr;
  *counters = nullptr;
  int n_cu = 0;
  if (int st = ellm::current_gfx950_device(device, &n_cu)) return st;
  const hipError_t prep = ellm::project_prepare();
  if (prep != hipSuccess) return ellm::set_error(ELLM_ERR_HIP, "projection kernels: %s", hipGetErrorString(prep));
  const size_t floats = ellm::project_workspace_floats(heads, K);
  if (floats * sizeof(float) > (size_t)64 << 20) return ELLM_OK;
  hipError_t e = hipMalloc((void**)ws, floats * sizeof(float));
  if (e == hipSuccess) e = hipMalloc((void**)counters, heads * sizeof(uint32_t));
  if (e == hipSuccess) e = hipMemset(*counters, 0, heads * sizeof(uint32_t));
  if (e != hipSuccess) {
    (void)hipFree(*ws);
    (void)hipFree(*counters);
    *ws = nullptr;
    *counters = nullptr;
    return ellm::set_error(ELLM_ERR_HIP, "projection workspace: %s", hipGetErrorString(e));
  }
  return ELLM_OK;
}
int free_small_workspace(float* ws, uint32_t* counters) {
  hipError_t e1 = ws ? hipFree(ws) : hipSuccess, e2 = counters ? hipFree(counters) : hipSuccess;
  if (e1 != hipSuccess || e2 != hipSuccess)
    return ellm::set_error(ELLM_ERR_HIP, "hipFree: %s", hipGetErrorString(e1 != hipSuccess ? e1 : e2));
  return ELLM_OK;
}
}  // namespace

extern "C" {

static int matmul3_create(const ellm_matmul3_desc* d, const ellm_kv_seq_table* table,
                          ellm_matmul3** out_handle) {
  if (!d || !out_handle) return ellm::set_error(ELLM_ERR_INVALID_ARGUMENT, "null descriptor or handle pointer");
  *out_handle = nullptr;
  ellm_matmul3_desc local;
  if (table) {
    if (!table->seq_offsets || !table->seq_capacity || !table->seq_capacity_host)
      return ellm::set_error(ELLM_ERR_INVALID_ARGUMENT, "the sequence table has a null member");
    if (d->batch_size == 0 || d->batch_size > table->sequences)
      return ellm::set_error(ELLM_ERR_OUT_OF_RANGE, "batch_size %zu, the sequence table has %zu entries",
                             d->batch_size, table->sequences);
    local = *d;
    size_t cap = 0;
    for (size_t i = 0; i < d->batch_size; ++i) {
      // (the kernels clamp a position to capacity - 1: a capacity of 0 would switch the clamp off)
      if (table->seq_capacity_host[i] == 0)
        return ellm::set_error(ELLM_ERR_INVALID_ARGUMENT, "sequence %zu of the table has capacity 0", i);
      cap = table->seq_capacity_host[i] > cap ? table->seq_capacity_host[i] : cap;
    }
    local.sequence_capacity = cap;   // the largest: per-sequence checks follow at run time
    d = &local;
  }
  const void* ptrs[] = {d->hidden, d->q_weight, d->k_weight, d->v_weight, d->q_state,
                        d->k_state, d->v_state, d->rope};
  for (const void* p : ptrs) {
    if (!p) return ellm::set_error(ELLM_ERR_INVALID_ARGUMENT, "hidden, weights, states and rope must be non-null device pointers");
    if (!aligned16(p)) return ellm::set_error(ELLM_ERR_INVALID_ARGUMENT, "hidden, weights, states and rope must be 16-byte aligned");
  }
  if (d->dtype != ELLM_DTYPE_F16 && d->dtype != ELLM_DTYPE_BF16)
    return ellm::set_error(ELLM_ERR_INVALID_ARGUMENT, "dtype %d is neither ELLM_DTYPE_F16 nor ELLM_DTYPE_BF16", d->dtype);
  if (d->head_size != 128)
    return ellm::set_error(ELLM_ERR_UNSUPPORTED, "head_size %zu: only 128 is supported", d->head_size);
  if (d->batch_size == 0 || d->attention_head_num == 0 || d->kv_head_num == 0 ||
      d->max_position_interval == 0 || d->sequence_capacity == 0)
    return ellm::set_error(ELLM_ERR_INVALID_ARGUMENT, "batch_size, head counts, max_position_interval, sequence_capacity must be > 0");
  if (d->hidden_size == 0 || d->hidden_size % 64 != 0 || d->hidden_size > kMaxK)
    return ellm::set_error(ELLM_ERR_UNSUPPORTED, "hidden_size %zu: must be a multiple of 64, at most %zu", d->hidden_size, kMaxK);
  if (d->kv_strides[3] != 1)
    return ellm::set_error(ELLM_ERR_INVALID_ARGUMENT, "kv_strides[3] must be 1 (head dimension contiguous)");
  for (int i = 0; i < 3; ++i)
    if (d->kv_strides[i] % 8 != 0)
      return ellm::set_error(ELLM_ERR_INVALID_ARGUMENT, "kv_strides[%d] = %zu is not a multiple of 8 elements", i, d->kv_strides[i]);
  if (d->rope_position_stride % 4 != 0 || d->rope_head_stride % 4 != 0 ||
      d->rope_position_stride > 0xffffffffu || d->rope_head_stride > 0xffffffffu)
    return ellm::set_error(ELLM_ERR_INVALID_ARGUMENT, "rope strides must be multiples of 4 elements below 2^32");
  if (d->rope_elems < 128)
    return ellm::set_error(ELLM_ERR_INVALID_ARGUMENT, "rope_elems %zu: the table holds less than one row", d->rope_elems);
  if (!(d->eps >= 0.0f) || !std::isfinite(d->eps))
    return ellm::set_error(ELLM_ERR_INVALID_ARGUMENT, "eps must be finite and >= 0");
  const size_t rows = d->max_position_interval * d->batch_size;
  if (rows > 0xffffffffu / 2 || d->attention_head_num > 4096 || d->kv_head_num > 4096)
    return ellm::set_error(ELLM_ERR_UNSUPPORTED, "too many rows or heads");
  ellm_matmul3* h = new (std::nothrow) ellm_matmul3;
  if (!h) return ellm::set_error(ELLM_ERR_HIP, "out of host memory");
  h->d = *d;
  h->seq_offsets = nullptr;
  h->seq_caps = nullptr;
  if (table) {
    h->seq_offsets = table->seq_offsets;
    h->seq_caps = table->seq_capacity;
    h->caps_host.assign(table->seq_capacity_host, table->seq_capacity_host + d->batch_size);
  }
  const int rc = alloc_small_workspace((uint32_t)(d->attention_head_num + 2 * d->kv_head_num),
                                       (uint32_t)d->hidden_size, &h->device, &h->ws, &h->counters);
  if (rc != ELLM_OK) {
    delete h;
    return rc;
  }
  *out_handle = h;
  return ELLM_OK;
}

int ellm_matmul3_create(const ellm_matmul3_desc* d, ellm_matmul3** out_handle) {
  return matmul3_create(d, nullptr, out_handle);
}

int ellm_matmul3_create_ragged(const ellm_matmul3_desc* d, const ellm_kv_seq_table* table,
                               ellm_matmul3** out_handle) {
  if (!table) return ellm::set_error(ELLM_ERR_INVALID_ARGUMENT, "null sequence table");
  return matmul3_create(d, table, out_handle);
}

int ellm_matmul3_reset(ellm_matmul3* h, void* stream) {
  if (!h) return ellm::set_error(ELLM_ERR_INVALID_ARGUMENT, "null handle");
  if (int st = ellm::check_current_device(h->device)) return st;
  if (!h->counters) return ELLM_OK;
  const hipError_t e = ellm::launch_fill_u32(h->counters, h->d.attention_head_num + 2 * h->d.kv_head_num, 0u,
                                             (hipStream_t)stream);
  if (e != hipSuccess) return ellm::set_error(ELLM_ERR_HIP, "counter reset launch: %s", hipGetErrorString(e));
  return ELLM_OK;
}

int ellm_matmul3_destroy(ellm_matmul3* h) {
  if (!h) return ELLM_OK;
  const int rc = free_small_workspace(h->ws, h->counters);
  delete h;
  return rc;
}

}  // extern "C"

int ellm::matmul3_fill_args(const ellm_matmul3* h, size_t position_index, size_t position_interval,
                            size_t batch_size, const uint32_t* positions, size_t max_start,
                            ellm::ProjectArgs* out) {
  const ellm_matmul3_desc& d = h->d;
  if (int st = ellm::check_current_device(h->device)) return st;
  if (position_interval > d.max_position_interval)
    return ellm::set_error(ELLM_ERR_OUT_OF_RANGE, "position_interval %zu exceeds max_position_interval %zu", position_interval, d.max_position_interval);
  if (batch_size > d.batch_size)
    return ellm::set_error(ELLM_ERR_OUT_OF_RANGE, "batch_size %zu exceeds the capacity %zu", batch_size, d.batch_size);
  const size_t last = (positions ? max_start : position_index) + position_interval - 1;
  if (last >= d.sequence_capacity)
    return ellm::set_error(ELLM_ERR_OUT_OF_RANGE, "position %zu is outside the cache (capacity %zu)", last, d.sequence_capacity);
  if (!positions)   // one shared range: it must fit every sequence written (per-sequence starts are clamped on the device)
    for (size_t i = 0; i < batch_size && i < h->caps_host.size(); ++i)
      if (last >= h->caps_host[i])
        return ellm::set_error(ELLM_ERR_OUT_OF_RANGE, "position %zu is outside sequence %zu (capacity %zu)", last, i, h->caps_host[i]);
  const size_t heads_max = d.attention_head_num > d.kv_head_num ? d.attention_head_num : d.kv_head_num;
  if (last * d.rope_position_stride + (heads_max - 1) * d.rope_head_stride + 128 > d.rope_elems)
    return ellm::set_error(ELLM_ERR_OUT_OF_RANGE, "position %zu is outside the rotary table (%zu elements)", last, d.rope_elems);
  ellm::ProjectArgs a{};
  a.x = d.hidden;
  a.w0 = d.q_weight;
  a.wk = d.k_weight;
  a.wv = d.v_weight;
  a.out0 = d.q_state;
  a.residual = nullptr;
  a.k_out = d.k_state;
  a.v_out = d.v_state;
  a.rope = d.rope;
  a.positions = positions;
  a.seq_offsets = h->seq_offsets;
  a.seq_caps = h->seq_caps;
  a.kv_stride_seq = d.kv_strides[0];
  a.kv_stride_head = d.kv_strides[1];
  a.kv_stride_pos = d.kv_strides[2];
  a.rope_pos_stride = (uint32_t)d.rope_position_stride;
  a.rope_head_stride = (uint32_t)d.rope_head_stride;
  a.K = (uint32_t)d.hidden_size;
  a.rows = (uint32_t)((position_interval - 1) * d.batch_size + batch_size);
  a.batch_pitch = (uint32_t)d.batch_size;
  a.batch = (uint32_t)batch_size;
  a.heads0 = (uint32_t)d.attention_head_num;
  a.heads_kv = (uint32_t)d.kv_head_num;
  a.position_index = (uint32_t)position_index;
  a.max_start = (uint32_t)max_start;
  a.finalize0 = 1;
  a.eps = d.eps;
  a.dtype = d.dtype;
  a.ws = h->ws;
  a.counters = h->counters;
  *out = a;
  return ELLM_OK;
}

extern "C" {

static int matmul3_launch(ellm_matmul3* h, size_t position_index, size_t position_interval,
                          size_t batch_size, const uint32_t* positions, size_t max_start,
                          void* stream) {
  if (position_interval == 0 || batch_size == 0) return ELLM_OK;
  ellm::ProjectArgs a{};
  if (int st = ellm::matmul3_fill_args(h, position_index, position_interval, batch_size, positions, max_start, &a))
    return st;
  const hipError_t e = ellm::launch_project(a, (hipStream_t)stream);
  if (e != hipSuccess) return ellm::set_error(ELLM_ERR_HIP, "projection launch: %s", hipGetErrorString(e));
  return ELLM_OK;
}

int ellm_matmul3_run(ellm_matmul3* h, size_t position_index, size_t position_interval,
                     size_t batch_size, void* stream) {
  if (!h) return ellm::set_error(ELLM_ERR_INVALID_ARGUMENT, "null handle");
  return matmul3_launch(h, position_index, position_interval, batch_size, nullptr, 0, stream);
}

int ellm_matmul3_run_ragged(ellm_matmul3* h, const uint32_t* positions, size_t max_position,
                            size_t batch_size, void* stream) {
  if (!h) return ellm::set_error(ELLM_ERR_INVALID_ARGUMENT, "null handle");
  if (!positions) return ellm::set_error(ELLM_ERR_INVALID_ARGUMENT, "positions must be a device array");
  return matmul3_launch(h, 0, 1, batch_size, positions, max_position, stream);
}

int ellm_projection_path(size_t rows, size_t heads, size_t k) {
  if (rows == 0 || heads == 0 || k == 0 || rows > 0xffffffffu / 2 || heads > 3 * 4096 || k > kMaxK)
    return -1;
  return ellm::project_path((uint32_t)rows, (uint32_t)heads, (uint32_t)k, true);
}

int ellm_matmul_add_create(const ellm_matmul_add_desc* d, ellm_matmul_add** out_handle) {
  if (!d || !out_handle) return ellm::set_error(ELLM_ERR_INVALID_ARGUMENT, "null descriptor or handle pointer");
  *out_handle = nullptr;
  const void* ptrs[] = {d->a, d->b_nt, d->residual, d->output};
  for (const void* p : ptrs) {
    if (!p) return ellm::set_error(ELLM_ERR_INVALID_ARGUMENT, "a, b_nt, residual and output must be non-null device pointers");
    if (!aligned16(p)) return ellm::set_error(ELLM_ERR_INVALID_ARGUMENT, "a, b_nt, residual and output must be 16-byte aligned");
  }
  if (d->dtype != ELLM_DTYPE_F16 && d->dtype != ELLM_DTYPE_BF16)
    return ellm::set_error(ELLM_ERR_INVALID_ARGUMENT, "dtype %d is neither ELLM_DTYPE_F16 nor ELLM_DTYPE_BF16", d->dtype);
  if (d->batch_size == 0 || d->max_position_interval == 0)
    return ellm::set_error(ELLM_ERR_INVALID_ARGUMENT, "batch_size and max_position_interval must be > 0");
  if (d->n == 0 || d->n % 128 != 0 || d->n > 128 * 4096)
    return ellm::set_error(ELLM_ERR_UNSUPPORTED, "n %zu: must be a multiple of 128, at most %d", d->n, 128 * 4096);
  if (d->k == 0 || d->k % 64 != 0 || d->k > kMaxK)
    return ellm::set_error(ELLM_ERR_UNSUPPORTED, "k %zu: must be a multiple of 64, at most %zu", d->k, kMaxK);
  if (d->max_position_interval * d->batch_size > 0xffffffffu / 2)
    return ellm::set_error(ELLM_ERR_UNSUPPORTED, "too many rows");
  ellm_matmul_add* h = new (std::nothrow) ellm_matmul_add;
  if (!h) return ellm::set_error(ELLM_ERR_HIP, "out of host memory");
  h->d = *d;
  const int rc = alloc_small_workspace((uint32_t)(d->n / 128), (uint32_t)d->k, &h->device, &h->ws, &h->counters);
  if (rc != ELLM_OK) {
    delete h;
    return rc;
  }
  *out_handle = h;
  return ELLM_OK;
}

int ellm_matmul_add_reset(ellm_matmul_add* h, void* stream) {
  if (!h) return ellm::set_error(ELLM_ERR_INVALID_ARGUMENT, "null handle");
  if (int st = ellm::check_current_device(h->device)) return st;
  if (!h->counters) return ELLM_OK;
  const hipError_t e = ellm::launch_fill_u32(h->counters, h->d.n / 128, 0u, (hipStream_t)stream);
  if (e != hipSuccess) return ellm::set_error(ELLM_ERR_HIP, "counter reset launch: %s", hipGetErrorString(e));
  return ELLM_OK;
}

int ellm_matmul_add_destroy(ellm_matmul_add* h) {
  if (!h) return ELLM_OK;
  const int rc = free_small_workspace(h->ws, h->counters);
  delete h;
  return rc;
}

int ellm_matmul_add_run(ellm_matmul_add* h, size_t position_index, size_t position_interval,
                        size_t batch_size, void* stream) {
  (void)position_index;  // as in the reference, the product does not depend on the position
  if (!h) return ellm::set_error(ELLM_ERR_INVALID_ARGUMENT, "null handle");
  const ellm_matmul_add_desc& d = h->d;
  if (position_interval == 0 || batch_size == 0) return ELLM_OK;
  if (int st = ellm::check_current_device(h->device)) return st;
  if (position_interval > d.max_position_interval)
    return ellm::set_error(ELLM_ERR_OUT_OF_RANGE, "position_interval %zu exceeds max_position_interval %zu", position_interval, d.max_position_interval);
  if (batch_size > d.batch_size)
    return ellm::set_error(ELLM_ERR_OUT_OF_RANGE, "batch_size %zu exceeds the capacity %zu", batch_size, d.batch_size);
  ellm::ProjectArgs a{};
  a.x = d.a;
  a.w0 = d.b_nt;
  a.wk = a.wv = nullptr;
  a.out0 = d.output;
  a.residual = d.residual;
  a.K = (uint32_t)d.k;
  a.rows = (uint32_t)((position_interval - 1) * d.batch_size + batch_size);
  a.batch_pitch = (uint32_t)d.batch_size;
  a.batch = (uint32_t)batch_size;
  a.heads0 = (uint32_t)(d.n / 128);
  a.heads_kv = 0;
  a.finalize0 = 0;
  a.dtype = d.dtype;
  a.ws = h->ws;
  a.counters = h->counters;
  const hipError_t e = ellm::launch_project(a, (hipStream_t)stream);
  if (e != hipSuccess) return ellm::set_error(ELLM_ERR_HIP, "projection launch: %s", hipGetErrorString(e));
  return ELLM_OK;
}

}  // extern "C"
