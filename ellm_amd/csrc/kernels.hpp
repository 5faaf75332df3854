// Internal interface between the C ABI (api.hip) and the kernel launchers.
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include "decode_plan.hpp"

struct ellm_attn_desc;

namespace ellm {

// Raw rows that the Q/K/V projection of a fused single-token step left for the attention
// kernels to finish: binary32 sums [part][sequence][column], column = head x 128 + element over
// the query heads, then the key heads, then the value heads.  A value is the sum of its `parts`
// (one or two) partial sums.  The attention kernels
// normalise and rotate the query and key heads while they load them and write the finished
// query rows, the new key row and the new value row to where the projection alone would have.
struct PendingRows {
  const float* raw;   // null: no raw sums pending
  uint32_t parts, part_stride, cols;   // part_stride, cols in floats
  const void* rope;   // (cos, sin) pairs, as in ProjectArgs
  uint32_t rope_pos_stride, rope_head_stride;
  float eps;
  // The other form (ellm_kv_append_attn_run; raw is null then): the query rows are final and
  // only the new key / value rows are pending, as stored 16-bit rows [sequence][kv_head][128]
  // that the cache write (kv_append_norm_rope_kernel) would normalise, rotate and copy: the
  // attention launch does that with the same arithmetic, bit for bit.  null: nothing of that
  // kind pending.
  const void* k_rows;
  const void* v_rows;
};

// Everything a launch needs; filled by the C ABI after validation.
struct AttnArgs {
  const void* q;
  const void* k;
  const void* v;
  void* out;
  float* lse;             // may be null
  uint32_t batch_pitch;   // sequences per token row of Q/O (capacity)
  uint32_t n_q_heads;
  uint32_t n_kv_heads;
  uint32_t group;         // n_q_heads / n_kv_heads
  size_t kv_stride_seq;   // elements
  size_t kv_stride_head;  // elements
  size_t kv_stride_pos;   // elements
  float scale;
  int dtype;              // 0 = binary16, 1 = bfloat16, 2 = binary32 (attn_general.hip only)
  uint32_t capacity;      // positions per K/V plane
  // per run
  uint32_t position_index;
  uint32_t position_interval;
  uint32_t batch;
  const uint32_t* positions;  // device, per sequence; null = position_index for all
  // caches whose sequences differ in capacity (both null otherwise): per-sequence element
  // offset of the first plane (replaces sequence x kv_stride_seq) and positions per plane
  const size_t* seq_offsets;
  const uint32_t* seq_caps;
  // single-token path workspace
  float* ws_acc;  // [sequence][query head][split][128]
  float* ws_ml;   // [sequence][query head][split][2]  (max in log2 units, sum)
  float* ws2_acc;      // second merge level: [sequence][query head][cluster][128]
  float* ws2_ml;
  uint32_t* counters;  // arrival counters, zero between launches
  uint32_t split_len;  // keys per split, multiple of 64
  uint32_t n_split;
  // chunk path, key range split over workgroups (may be null: never split): room for
  // prefill_part_rows partial rows of 128 + 2 floats
  float* prefill_part_o;
  float* prefill_part_ml;
  size_t prefill_part_rows;
  uint32_t n_cu;
  PendingRows pending;   // single-token path only
};
// Partial rows the chunk path's workspace holds for an operator of this shape (0: none needed).
size_t prefill_workspace_rows(uint32_t max_interval, uint32_t batch_capacity, uint32_t n_q_heads,
                              uint32_t n_cu);

hipError_t launch_decode(const AttnArgs& a, hipStream_t stream);
// Per-sequence positions, the planes' keys dealt evenly to `wgs` workgroups (decode_balanced.hip):
// whether a call of this shape goes there, and the launch (a.positions must be set).
bool decode_balanced_takes(const DecodeWorkspace& w, uint32_t batch, uint32_t n_kv_heads, uint32_t group,
                           uint32_t max_len, uint32_t wgs);
hipError_t launch_decode_balanced(const AttnArgs& a, uint32_t wgs, hipStream_t stream);
hipError_t launch_prefill(const AttnArgs& a, hipStream_t stream);
// Any head size up to 256 and binary32 storage (dtype 2): chunk and single-token calls alike.
hipError_t launch_attn_general(const AttnArgs& a, uint32_t head_size, hipStream_t stream);

// Where the rows of a cache layer live: plane of (sequence, head) at
// seq_plane_offset(seq_offsets, stride_seq, sequence) + head x stride_head, rows 128 apart;
// seq_caps (may be null) bounds the positions written per sequence on the device.
struct KvLayout {
  size_t stride_seq, stride_head;
  const size_t* seq_offsets;
  const uint32_t* seq_caps;
};
hipError_t launch_kv_append(void* k_dst, void* v_dst, const void* k_src, const void* v_src,
                            uint32_t n_tokens, uint32_t batch, uint32_t src_batch_pitch,
                            uint32_t n_kv_heads, const KvLayout& layout, uint32_t position_index,
                            hipStream_t stream);

// Same, with RMS norm and rotary rotation of the key rows; rope: [positions][128] of
// the cache's type, (cos, sin) interleaved; positions (may be null): per-sequence start
// positions on the device, each clamped to max_start.
hipError_t launch_kv_append_norm_rope(void* k_dst, void* v_dst, const void* k_src,
                                      const void* v_src, const void* rope,
                                      const uint32_t* positions, uint32_t n_tokens, uint32_t batch,
                                      uint32_t src_batch_pitch, uint32_t n_kv_heads,
                                      const KvLayout& layout, uint32_t position_index,
                                      uint32_t max_start, float eps, int dtype,
                                      hipStream_t stream);

hipError_t launch_positions_advance(uint32_t* positions, uint32_t n, uint32_t by,
                                    hipStream_t stream);
// p[i] = value for i < n: a kernel, not a memset node, so that it can be recorded into a graph.
hipError_t launch_fill_u32(uint32_t* p, size_t n, uint32_t value, hipStream_t stream);

// Projection C = X . W^T on MFMA with the per-head epilogue (see project.hip).
// Column segment 0 (heads0 heads, weights w0) goes row-major to out0 [rows][heads0 * 128],
// optionally normalised + rotated (finalize0) and with `residual` added; segments 1 and 2
// (heads_kv heads each, weights wk / wv) go to token coordinates of k_out / v_out through
// the three strides, the key rows normalised + rotated.  Row r of X is token r / batch_pitch
// of sequence r % batch_pitch; sequences >= batch are skipped.
struct ProjectArgs {
  const void* x;
  const void* w0;
  const void* wk;
  const void* wv;
  void* out0;
  const void* residual;
  void* k_out;
  void* v_out;
  const void* rope;
  const uint32_t* positions;
  const size_t* seq_offsets;   // as in AttnArgs (null: sequence x kv_stride_seq)
  const uint32_t* seq_caps;
  size_t kv_stride_seq, kv_stride_head, kv_stride_pos;
  uint32_t rope_pos_stride, rope_head_stride;
  uint32_t K, rows, batch_pitch, batch, heads0, heads_kv;
  uint32_t position_index, max_start, finalize0;
  float eps;
  int dtype;
  // workspace of the few-rows kernel (may be null: the tile kernel runs whatever the row count)
  float* ws;
  uint32_t* counters;
  // raw_out: the few-rows kernel leaves the binary32 sums of every column in ws, laid out as
  // PendingRows describes (one part), and writes nothing else (requires project_raw_takes())
  uint32_t raw_out;
};
// Whether a projection of this shape can leave raw rows (the few-rows kernel takes it).
bool project_raw_takes(uint32_t rows, uint32_t heads, uint32_t K, bool has_workspace);
hipError_t launch_project(const ProjectArgs& a, hipStream_t stream);
// Few-rows kernel: rows it handles at most, floats of partial sums and counters it needs.
size_t project_workspace_floats(uint32_t heads, uint32_t K);
// The kernel a projection of this shape runs (heads = 128-wide output column groups).
enum { kPathFewRows = 0, kPathTiles128 = 1, kPathTiles256x1 = 2, kPathTiles = 3 };
int project_path(uint32_t rows, uint32_t heads, uint32_t K, bool has_workspace);
// Per-device set-up of the projection kernels (LDS limits); call with the device current.
hipError_t project_prepare();

// The current device and its compute-unit count.  ELLM_ERR_NO_DEVICE (message recorded) when
// there is none or it is not a gfx950 part.
int current_gfx950_device(int* device, int* n_cu);
// ELLM_OK when `device` (the one a handle was created on) is the calling thread's current
// device; a handle's workspace and the caller's buffers live on that device only.
int check_current_device(int device);

// The checks ellm_attn_create applies to a description (status + message recorded), and the
// shape part of AttnArgs taken from a checked description (workspace pointers left null).
int validate_attn_desc(const ellm_attn_desc* d);
// A description the MFMA kernels do not take (head size other than 128, or binary32 storage):
// its calls go to launch_attn_general.
bool attn_is_general(const ellm_attn_desc& d);
void attn_args_from_desc(const ellm_attn_desc& d, AttnArgs* a);

// Looks up, once per device, the address of the current device's copy of the static scratch
// that ellm_attn_run_noalloc uses (noalloc.hip).
void prepare_static_scratch();

// Records the message ellm_last_error_string() returns on this thread; returns status.
int set_error(int status, const char* fmt, ...) __attribute__((format(printf, 2, 3)));

}  // namespace ellm
