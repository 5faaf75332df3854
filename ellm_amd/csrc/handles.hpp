// The operator handles behind the C ABI and the internal entry points that more than one
// source file needs (api.hip: attention; project_api.hip: projections; step.hip: the fused
// single-token step that drives both).
#pragma once

#include <vector>

#include "../../include/ellm_attn.h"
#include "kernels.hpp"

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
  // sequences of different capacities (ellm_attn_create_ragged): device tables (borrowed from
  // the cache) and a host copy of the capacities for the range checks; empty / null otherwise
  const size_t* seq_offsets;
  const uint32_t* seq_caps;
  std::vector<size_t> caps_host;
  // a head size other than 128 or binary32 storage: every call goes to attn_general.hip
  bool general;
};

struct ellm_matmul3 {
  ellm_matmul3_desc d;
  int device;
  float* ws;
  uint32_t* counters;
  // destination with per-sequence capacities (ellm_matmul3_create_ragged); null / empty otherwise
  const size_t* seq_offsets;
  const uint32_t* seq_caps;
  std::vector<size_t> caps_host;
};
namespace ellm {

// AttnArgs of a handle: its description, workspace and sequence tables (per-run fields unset).
void attn_fill_args(const ellm_attn* h, AttnArgs* a);
// The single-token launch of a handle (a->batch, a->position_index, a->positions, a->pending set):
// the kernel for sequences of different lengths when the call is large enough, else the split plan.
int attn_run_single_token(ellm_attn* h, AttnArgs* a, uint32_t max_position, hipStream_t stream);

// The range checks of ellm_matmul3_run / _run_ragged and the launch arguments of a call
// (ELLM_OK, or a status with the message recorded).
int matmul3_fill_args(const ellm_matmul3* h, size_t position_index, size_t position_interval,
                      size_t batch_size, const uint32_t* positions, size_t max_start, ProjectArgs* a);

}  // namespace ellm
