// The Q/K/V projection and the attention of a single-token step as one call
// (ellm_matmul3_attn_run / _run_ragged, declared in include/ellm_attn.h).
//
// Run one after the other, ellm_matmul3_run finishes every query and key head row inside its
// own launch: the 128 columns of a head are spread over several workgroups, so the row's sum
// of squares needs an exchange between workgroups (partial sums to memory, an arrival count,
// the last one reads the head back), which is a quarter of a launch that only streams 21 MB
// of weights.  Fused, the projection leaves the raw binary32 sums of every column in its
// workspace and ends; the attention kernel that follows normalises and rotates the query rows
// while it loads them (it has to read them anyway), and the workgroup that holds a plane's
// last key does the same for the new key row, copies the new value row, writes both to the
// cache and takes them as one more chunk of its stream.  After the call q_state, the caches
// and the attention output hold what the two separate calls leave there (reference:
// MatMul3::run, src/compiler/mul/matmul3.rs:289-385, then Attention::run,
// src/compiler/mul/attention.rs:69-156, consecutive operators of one layer in
// src/qwen3_moe/attention.rs:126-174).
#include <hip/hip_runtime.h>

#include "handles.hpp"

namespace {

// Why a pair of handles cannot run fused (null: it can).
const char* mismatch(const ellm_matmul3* m, const ellm_attn* a) {
  const ellm_matmul3_desc& p = m->d;
  const ellm_attn_desc& d = a->desc;
  if (m->device != a->device) return "the handles were created on different devices";
  if (a->general) return "the attention operator has a head size other than 128 or binary32 storage";
  if (p.q_state != d.q) return "the projection's q_state is not the attention operator's q";
  if (p.k_state != d.k || p.v_state != d.v) return "the projection's k_state / v_state are not the attention operator's k / v";
  if (p.dtype != d.dtype) return "the handles differ in dtype";
  if (p.batch_size != d.batch_size) return "the handles differ in batch_size (the row pitch of q)";
  if (p.attention_head_num != d.attention_head_num || p.kv_head_num != d.kv_head_num)
    return "the handles differ in head counts";
  for (int i = 0; i < 4; ++i)
    if (p.kv_strides[i] != d.kv_strides[i] && !(i == 0 && m->seq_offsets)) return "the handles differ in kv_strides";
  if (m->seq_offsets != a->seq_offsets || m->seq_caps != a->seq_caps)
    return "the handles were created with different sequence tables";
  if (p.sequence_capacity != d.sequence_capacity) return "the handles differ in sequence_capacity";
  return nullptr;
}

bool fused_takes(const ellm_matmul3* m, size_t batch_size) {
  const ellm_matmul3_desc& p = m->d;
  return ellm::project_raw_takes((uint32_t)batch_size, (uint32_t)(p.attention_head_num + 2 * p.kv_head_num),
                                 (uint32_t)p.hidden_size, m->ws && m->counters);
}

int run(ellm_matmul3* m, ellm_attn* a, size_t position_index, const uint32_t* positions, size_t max_position,
        size_t batch_size, void* stream) {
  if (!m || !a) return ellm::set_error(ELLM_ERR_INVALID_ARGUMENT, "null handle");
  if (batch_size == 0) return ELLM_OK;
  if (const char* why = mismatch(m, a)) return ellm::set_error(ELLM_ERR_INVALID_ARGUMENT, "%s", why);
  if (!fused_takes(m, batch_size)) {
    // shapes the few-rows projection does not take: the two ordinary calls, same results
    const int st = positions ? ellm_matmul3_run_ragged(m, positions, max_position, batch_size, stream)
                             : ellm_matmul3_run(m, position_index, 1, batch_size, stream);
    if (st != ELLM_OK) return st;
    return positions ? ellm_attn_run_ragged(a, positions, max_position, batch_size, stream)
                     : ellm_attn_run(a, position_index, 1, batch_size, stream);
  }
  const size_t bound = positions ? max_position : position_index;
  ellm::ProjectArgs pa{};
  if (int st = ellm::matmul3_fill_args(m, position_index, 1, batch_size, positions, max_position, &pa)) return st;
  // the attention operator's own range checks (ellm_attn_run / ellm_attn_run_ragged)
  if (batch_size > a->desc.batch_size || bound >= a->desc.sequence_capacity)
    return ellm::set_error(ELLM_ERR_OUT_OF_RANGE, "batch_size %zu / position %zu outside the attention operator's %zu / %zu",
                           batch_size, bound, a->desc.batch_size, a->desc.sequence_capacity);
  pa.raw_out = 1;
  hipError_t e = ellm::launch_project(pa, (hipStream_t)stream);
  if (e != hipSuccess) return ellm::set_error(ELLM_ERR_HIP, "projection launch: %s", hipGetErrorString(e));

  ellm::AttnArgs aa;
  ellm::attn_fill_args(a, &aa);
  aa.position_index = (uint32_t)bound;
  aa.position_interval = 1;
  aa.batch = (uint32_t)batch_size;
  aa.positions = positions;
  aa.pending.raw = m->ws;
  aa.pending.parts = 1;
  aa.pending.cols = (uint32_t)((m->d.attention_head_num + 2 * m->d.kv_head_num) * 128);
  aa.pending.part_stride = 0;
  aa.pending.rope = m->d.rope;
  aa.pending.rope_pos_stride = (uint32_t)m->d.rope_position_stride;
  aa.pending.rope_head_stride = (uint32_t)m->d.rope_head_stride;
  aa.pending.eps = m->d.eps;
  return ellm::attn_run_single_token(a, &aa, (uint32_t)bound, (hipStream_t)stream);
}

}  // namespace

extern "C" {

int ellm_matmul3_attn_run(ellm_matmul3* proj, ellm_attn* attn, size_t position_index, size_t batch_size,
                          void* stream) {
  return run(proj, attn, position_index, nullptr, 0, batch_size, stream);
}

int ellm_matmul3_attn_run_ragged(ellm_matmul3* proj, ellm_attn* attn, const uint32_t* positions,
                                 size_t max_position, size_t batch_size, void* stream) {
  if (!positions) return ellm::set_error(ELLM_ERR_INVALID_ARGUMENT, "positions must be a device array");
  return run(proj, attn, 0, positions, max_position, batch_size, stream);
}

int ellm_matmul3_attn_path(const ellm_matmul3* proj, const ellm_attn* attn, size_t batch_size) {
  if (!proj || !attn) return -ellm::set_error(ELLM_ERR_INVALID_ARGUMENT, "null handle");
  if (const char* why = mismatch(proj, attn)) return -ellm::set_error(ELLM_ERR_INVALID_ARGUMENT, "%s", why);
  if (batch_size == 0 || batch_size > proj->d.batch_size)
    return -ellm::set_error(ELLM_ERR_OUT_OF_RANGE, "batch_size %zu outside the handles' %zu", batch_size,
                            proj->d.batch_size);
  return fused_takes(proj, batch_size) ? 1 : 0;
}

}  // extern "C"
