/*
 * ellm_attn.h — C ABI of the MI355X (gfx950) attention path for eLLM.
 *
 * What this replaces in the reference (paths relative to the eLLM tree):
 *   - compiler::mul::attention::Attention::{new,run}   src/compiler/mul/attention.rs:41-67, 69-156
 *   - its leaf kernels                                 src/kernel/x86_64/f16_512/flash_attention.rs:30-92
 *                                                      src/kernel/generic/flash_attention.rs:60-89
 *   - the per-layer key/value buffers of memory::Cache src/memory/cache.rs:23, 69-75
 *
 * All pointers named "device" are HIP device pointers.  Every function returns
 * ELLM_OK (0) or an ellm_status; nothing aborts the process.  Functions taking a
 * stream enqueue work on it and return without waiting (stream = NULL is the
 * HIP null stream).  A handle may be used from one host thread at a time, and
 * ONE LAUNCH OF A HANDLE MAY BE IN FLIGHT AT A TIME: a handle's workspace (split
 * partials, arrival counters) is shared by all its runs, so runs of one handle
 * on two streams, or two graphs recorded from one handle replayed at once, race
 * and give wrong results; runs in stream order do not.  The arrival counters are
 * zero between launches (the kernels put them back); a launch that was killed
 * half-way leaves them counting, and ellm_*_reset puts them right.  A
 * handle (operator, cache, projection) belongs to the device that was current
 * when it was created: its workspace lives there, and a run or append called
 * while another device is current returns ELLM_ERR_INVALID_ARGUMENT.
 *
 * Only head_size == 128 and 16-bit storage (binary16 / bfloat16) are supported,
 * like the reference's AVX-512 kernel (head_size hard-wired to 128 there,
 * flash_attention.rs:51-56).  Scores, soft-max state and output accumulation are
 * binary32.
 */
#ifndef ELLM_ATTN_H_
#define ELLM_ATTN_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum ellm_status {
  ELLM_OK = 0,
  ELLM_ERR_INVALID_ARGUMENT = 1, /* null pointer, zero size, bad dtype, strides, ... */
  ELLM_ERR_UNSUPPORTED = 2,      /* head_size beyond 256, != 128 for projections and caches, ... */
  ELLM_ERR_OUT_OF_RANGE = 3,     /* position / batch / slot beyond the stated capacity */
  ELLM_ERR_HIP = 4,              /* a HIP runtime call (or a host allocation) failed      */
  ELLM_ERR_NO_DEVICE = 5         /* no gfx950 device visible                           */
} ellm_status;

typedef enum ellm_dtype {
  ELLM_DTYPE_F16 = 0,
  ELLM_DTYPE_BF16 = 1,
  ELLM_DTYPE_F32 = 2  /* attention only (ellm_attn_create / _create_ragged), see ellm_attn_desc */
} ellm_dtype;

/* Message for the last non-OK status returned on the calling thread. */
const char* ellm_last_error_string(void);

/* Library version (major*10000 + minor*100 + patch). */
int ellm_attn_version(void);

/* Number of visible devices this library can run on (gfx950); 0 when none.
 * Never fails: returns 0 on any HIP error. */
int ellm_device_count(void);

/* ------------------------------------------------------------------------ *
 * Attention operator
 * ------------------------------------------------------------------------ */

/*
 * Mirrors the argument list of Attention::new (src/compiler/mul/attention.rs:41-54)
 * as called from Tensor::attention (src/ptensor/tensor.rs:123-135):
 *
 *   q, out : device, [position_interval][batch_capacity][attention_head_num][head_size],
 *            row-major (src/compiler/mul/attention.rs:78, 116-119).
 *   k, v   : device, viewed as [sequence][kv_head][position][head_size] through
 *            kv_strides (elements): kv_strides[0] per sequence, [1] per kv head,
 *            [2] per position, [3] must be 1.  The dimension-first cache of this
 *            library has kv_strides = {kv_heads*capacity*128, capacity*128, 128, 1}.
 *   inverse_sqrt_head : soft-max scale applied to q.k (attention.rs:52, 66).
 *
 * Additions the reference does not have:
 *   lse    : optional device [position_interval][batch_capacity][attention_head_num]
 *            float, receives log(sum_j exp(scale * q.k_j)) per query row.
 *   dtype, sequence_capacity (positions per K/V plane; run() rejects positions
 *            at or beyond it), max_position_interval (largest position_interval
 *            run() will be given; sizes q/out).
 *
 * head_size 128 with 16-bit storage (every model configuration the reference ships) runs the
 * MFMA kernels.  Any other head_size from 1 to 256, and ELLM_DTYPE_F32 storage (the type of
 * the reference's generic leaf and of its operator test, src/kernel/generic/
 * flash_attention.rs:60-89, src/compiler/mul/attention.rs:262-330), run a plain kernel with the
 * same arguments, masks and results (binary32 arithmetic throughout), written to be right and
 * not for a roofline; there kv_strides[0..2] need not be multiples of 8.
 * ellm_attn_run_noalloc and ellm_matmul3_attn_run take 128-wide 16-bit heads only.
 */
typedef struct ellm_attn_desc {
  const void* q;
  const void* k;
  const void* v;
  void* out;
  float* lse; /* may be NULL */
  size_t batch_size; /* capacity in sequences: the Q/O row pitch, as in the reference */
  size_t attention_head_num;
  size_t kv_head_num;
  size_t head_size;
  size_t kv_strides[4];
  float inverse_sqrt_head;
  int dtype; /* ellm_dtype */
  size_t sequence_capacity;
  size_t max_position_interval;
} ellm_attn_desc;

typedef struct ellm_attn ellm_attn;

/* Validates the description and allocates the operator's own workspace (split
 * partial results for the single-token path and, when max_position_interval > 1,
 * for short chunks on long caches: at most 68 MB).  Borrowed pointers are not owned. */
int ellm_attn_create(const ellm_attn_desc* desc, ellm_attn** out_handle);

/* Frees the handle and its workspace only.  NULL is accepted. */
int ellm_attn_destroy(ellm_attn* handle);

/* Puts the handle's arrival counters back to zero, in stream order (a small fill kernel: it
 * may be recorded into a graph).  Only needed after a launch of this handle did not run to
 * its end (a killed process sharing the memory, a device reset survived by the allocation);
 * no counterpart in the reference. */
int ellm_attn_reset(ellm_attn* handle, void* stream);

/*
 * Attention::run (src/compiler/mul/attention.rs:69-76) without the cpu_num /
 * thread_id pair: queries at positions [position_index, position_index +
 * position_interval) of the first batch_size sequences; the query at position p
 * attends to keys 0..=p of its own sequence (flash_attention.rs:57-58).
 * position_interval == 1 takes the split-KV single-token kernel, larger
 * intervals the tiled MFMA kernel (with the key range split over workgroups and
 * a merge launch behind it when the call has too few query rows to fill the
 * device; calls with at most 384 query rows per K/V plane on 512 keys or more
 * take a kernel that streams every plane once).  Zero batch_size or
 * position_interval is a no-op returning ELLM_OK.  One run of a handle in flight
 * at a time (see the top of this file).
 * K/V rows at positions up to position_index + position_interval - 1 must hold finite
 * values: a query row multiplies the value rows of the chunk's later tokens by a
 * probability of exactly 0, and 0 x infinity is not 0 (the reference never reads them;
 * rows beyond the call's last position are never read here either).
 */
int ellm_attn_run(ellm_attn* handle, size_t position_index, size_t position_interval,
                  size_t batch_size, void* stream);

/*
 * Single-token step with one position per sequence (the reference has a single
 * shared position_index, which cannot express sequences of different lengths).
 * positions: device, batch_size uint32 values; sequence i attends to keys
 * 0..=positions[i].  max_position: an upper bound (inclusive) on every entry,
 * known on the host; it sizes the launch.  Entries above max_position or at or
 * beyond sequence_capacity are clamped to that bound on the device.
 * Large calls (see ellm_attn_ragged_path) deal the keys of all K/V planes to the
 * workgroups in equal shares, so that the time follows the sum of the lengths and
 * not the longest of them; the split of the work depends on the positions only,
 * hence equal positions give equal bits.
 */
int ellm_attn_run_ragged(ellm_attn* handle, const uint32_t* positions, size_t max_position,
                         size_t batch_size, void* stream);

/*
 * Which kernel ellm_attn_run_ragged runs for a call with this max_position and batch_size
 * on this handle: 0 = the single-token kernel of ellm_attn_run (every K/V plane split alike,
 * sized for max_position), 1 = the kernel that deals the keys of all planes to the workgroups
 * in equal shares, whatever the sequences' lengths (taken when the call is large enough for
 * the split to matter); negative: a status code (null handle, arguments out of range).  No
 * counterpart in the reference (its Attention::run has one code path); it lets a test or a
 * harness see which kernel its shapes reach.
 */
int ellm_attn_ragged_path(const ellm_attn* handle, size_t max_position, size_t batch_size);

/*
 * The single-token step of ellm_attn_run / ellm_attn_run_ragged (position_interval == 1)
 * without a handle and without any allocation.  No counterpart in the reference: it is
 * for callers that cannot call hipMalloc — code under HIP graph capture, tight serving
 * loops, harnesses that forbid allocation.  The description is read on every call (q, k,
 * v, out, lse, strides, scale as for ellm_attn_create; max_position_interval is ignored
 * beyond its range check); nothing is created and nothing needs destroying.
 *   positions == NULL : every sequence attends to keys 0..=position;
 *   positions != NULL : device uint32[batch_size], one position per sequence, each
 *                       clamped to `position` (their upper bound, which sizes the launch).
 * Same kernel and split plan as ellm_attn_run and as the ellm_attn_run_ragged calls for which
 * ellm_attn_ragged_path returns 0, so those results are bit-identical (the kernel for large
 * calls with per-sequence positions, path 1, splits the keys differently: same tolerance,
 * other bits).
 * The split partials and arrival counters live in a static device array of 5,074,944
 * bytes that every device the library runs on holds until the process ends; the call
 * uses the current device's copy.  Limit: sequences x query heads x splits <= 8192
 * partial rows, which covers GQA groups of up to 16 query heads on a 256-unit part
 * (every split plan inside that limit also fits the cluster partials and the counters);
 * larger shapes return ELLM_ERR_OUT_OF_RANGE, the message naming the bound, and must use
 * a handle.  Every call on a
 * device shares that device's array: calls that overlap on one device (two streams, or
 * two graphs replayed at once) race; calls in stream order do not.  It calls no
 * hipMalloc / hipFree and launches kernels only (the counters are cleared by a small
 * fill kernel), so it may be recorded into a graph.  The first call on a device looks up
 * the array's address and the device's properties (later calls only ask which device is
 * current): that first call must happen outside a stream capture, or after any
 * ellm_attn_create / ellm_kv_create on that device, which do
 * the lookup themselves.
 */
int ellm_attn_run_noalloc(const ellm_attn_desc* desc, const uint32_t* positions, size_t position,
                          size_t batch_size, void* stream);

/* ------------------------------------------------------------------------ *
 * Key/value cache: one allocation, [layer][sequence][kv_head][position][128],
 * for keys and one for values, written in place at token coordinates.
 * Replaces the per-layer "key_position_tensor" / "value_tensor" buffers of
 * memory::Cache (src/memory/cache.rs:23, 69-75) and the 64-byte aligned,
 * zero-filled, never-moved allocation of src/memory/allocator.rs:4-27.
 * ------------------------------------------------------------------------ */

typedef struct ellm_kv_cache ellm_kv_cache;

typedef struct ellm_kv_desc {
  size_t layers;
  size_t sequences;  /* slots */
  size_t kv_head_num;
  size_t head_size;  /* 128 */
  size_t capacity;   /* positions per plane */
  int dtype;         /* ellm_dtype */
} ellm_kv_desc;

/* Allocates and zero-fills both tensors on the current device. */
int ellm_kv_create(const ellm_kv_desc* desc, ellm_kv_cache** out_cache);
int ellm_kv_destroy(ellm_kv_cache* cache);

/* Device base pointers of one layer's K and V ([sequence][kv_head][position][128])
 * and the four element strides to hand to ellm_attn_desc.kv_strides. */
int ellm_kv_layer(const ellm_kv_cache* cache, size_t layer, void** k, void** v,
                  size_t kv_strides[4]);

/*
 * A cache whose sequences (slots) have different capacities: still static, non-paged and
 * contiguous per (layer, kv head, sequence) plane, offsets computed once at creation.
 * Layout [layer][kv_head][sequence: its own positions][128]: the plane of (sequence s,
 * head h) starts at  layer base + 128 * (positions of the sequences before s) +
 * h * kv_strides[1].  A mixed step over 33 sequences of 16384 ... 131072 positions x 48
 * layers then takes what the sequences need (~220 GB) instead of 33 x 131072 positions a
 * layer (425 GB).  Same concept as the uniform cache (static max-shape K/V addressed by
 * coordinates, README.md:51-54; per-layer persistent buffers, src/memory/cache.rs:23,
 * 69-75); the reference itself has one capacity for every sequence.
 * ellm_kv_append / ellm_kv_append_norm_rope work on both kinds of cache (a call with one
 * shared position range must fit the shortest of the sequences it writes).
 */
typedef struct ellm_kv_ragged_desc {
  size_t layers;
  size_t sequences;
  size_t kv_head_num;
  size_t head_size;         /* 128 */
  const size_t* capacities; /* host, [sequences]: positions per plane of each sequence, > 0 */
  int dtype;                /* ellm_dtype */
} ellm_kv_ragged_desc;
int ellm_kv_create_ragged(const ellm_kv_ragged_desc* desc, ellm_kv_cache** out_cache);

/* Where the sequences [first_sequence, ...) of such a cache start and how many positions
 * each holds: what the operators need beside the strides.  The arrays belong to the cache
 * and live as long as it does. */
typedef struct ellm_kv_seq_table {
  const size_t* seq_offsets;        /* device: element offset of each sequence's first plane */
  const uint32_t* seq_capacity;     /* device: positions per plane of each sequence */
  const size_t* seq_capacity_host;  /* host copy of the capacities */
  size_t sequences;                 /* entries in each array */
} ellm_kv_seq_table;

/* ellm_kv_layer for a cache with per-sequence capacities.  kv_strides[1..3] are the head,
 * position and element strides; kv_strides[0] has no meaning (every sequence has its own
 * offset in the table) and is only there to keep the four-stride shape.  Hand k, v,
 * kv_strides and the table to ellm_attn_create_ragged / ellm_matmul3_create_ragged:
 * their sequence i is the cache's sequence first_sequence + i. */
int ellm_kv_layer_ragged(const ellm_kv_cache* cache, size_t layer, size_t first_sequence, void** k,
                         void** v, size_t kv_strides[4], ellm_kv_seq_table* table);

/* ellm_attn_create on such a layer: sequence i's planes start at k + seq_offsets[i] +
 * head * kv_strides[1]; desc->kv_strides[0] and desc->sequence_capacity are ignored (the
 * capacity is per sequence: a run with one shared position range must fit every sequence it
 * covers, per-sequence positions are clamped to each sequence's own capacity on the
 * device).  desc->batch_size may not exceed table->sequences.  run / run_ragged / destroy
 * as for any handle. */
int ellm_attn_create_ragged(const ellm_attn_desc* desc, const ellm_kv_seq_table* table,
                            ellm_attn** out_handle);

/*
 * Writes n_tokens new positions [position_index, position_index + n_tokens) of
 * sequences [0, batch_size) of one layer.  k_src / v_src: device,
 * [n_tokens][src_batch_pitch][kv_head_num][128] — the layout in which the
 * projection produces them (src/qwen3_moe/attention.rs:142-166, before its
 * permute).  src_batch_pitch is the source's sequence capacity (>= batch_size).
 */
int ellm_kv_append(ellm_kv_cache* cache, size_t layer, size_t position_index, size_t n_tokens,
                   size_t batch_size, const void* k_src, const void* v_src,
                   size_t src_batch_pitch, void* stream);

/*
 * ellm_kv_append with the key rows normalised and rotated on the way into the
 * cache; value rows are copied as they are.  Per 128-wide key row x of a token
 * at position p:
 *     y = x / (sqrt(mean(x^2)) + eps)                 (RMS norm, weight 1: eps is
 *                                                     added to the root mean square,
 *                                                     src/kernel/generic/rms_norm.rs:6-26)
 *     (k[2j], k[2j+1]) = (y[2j] c - y[2j+1] s, y[2j] s + y[2j+1] c),
 *                        (c, s) = (rope[p][2j], rope[p][2j+1])
 *                                                    (src/kernel/generic/complex_mul.rs:3-20)
 * which is what the reference's fused projection applies to every finished
 * head column (matmul_finalize_rmsnorm_rope_inplace_3x128,
 * src/kernel/x86_64/f16_512/matmul_rms_complex.rs:76-96, called from
 * src/compiler/mul/matmul3.rs:243-254 with eps = 1e-6, :436-451), written
 * straight to token coordinates as the reference's output_to_kv flag intends
 * (src/compiler/zip_map/complex_zip.rs:92-100: destination moved by the
 * position, rotary row advanced one head_size per position).  Arithmetic is
 * binary32, rounded to the storage type once.
 *
 * rope: device, [rope_positions][128] in the cache's dtype, (cos, sin)
 * interleaved — the reference's "model.position_embedding.weight",
 * [max_position_embeddings][1][1][head_size] (src/qwen3_moe/attention.rs:258-262).
 * positions: NULL (every sequence starts at position_index) or device
 * uint32[batch_size] start positions, one per sequence, for single-token steps
 * over sequences of different lengths; max_position bounds them (larger
 * entries are clamped to it) and is what the range checks use.
 */
int ellm_kv_append_norm_rope(ellm_kv_cache* cache, size_t layer, size_t position_index,
                             size_t n_tokens, size_t batch_size, const void* k_src,
                             const void* v_src, size_t src_batch_pitch, const void* rope,
                             size_t rope_positions, float eps, const uint32_t* positions,
                             size_t max_position, void* stream);

/*
 * ellm_kv_append_norm_rope for one new token per sequence and the attention over the cache
 * including that token (ellm_attn_run / ellm_attn_run_ragged with position_interval 1), as one
 * launch: the workgroup of the attention kernel that holds a plane's last key normalises and
 * rotates the new key row (the cache write's own arithmetic: the row in the cache carries the
 * same bits), copies the new value row, writes both to the cache and takes them as the last
 * key of its stream.  For callers that run their own projection and keep the two steps apart
 * otherwise: a single-token step of a layer is then one launch instead of two (the reference
 * does the write inside its projection, src/compiler/mul/matmul3.rs:243-254, and runs the
 * attention operator next, src/qwen3_moe/attention.rs:126-174; with this library's projection
 * the corresponding call is ellm_matmul3_attn_run).
 * attn must have been created over this layer of this cache (k, v, kv_strides of ellm_kv_layer /
 * ellm_kv_layer_ragged from the cache's first sequence, the cache's dtype); else
 * ELLM_ERR_INVALID_ARGUMENT.  k_src, v_src: device, [batch_size][kv_head][128] rows of the new
 * token; rope, rope_positions, eps, positions, max_position as in ellm_kv_append_norm_rope.
 * The query rows in the operator's q are final (normalised and rotated by the caller's
 * projection).  Results: the cache as ellm_kv_append_norm_rope leaves it, out / lse as
 * ellm_attn_run leaves them (same tolerance; the new key is taken in a different chunk).
 */
int ellm_kv_append_attn_run(ellm_kv_cache* cache, size_t layer, ellm_attn* attn, size_t position_index,
                            size_t batch_size, const void* k_src, const void* v_src, const void* rope,
                            size_t rope_positions, float eps, void* stream);
int ellm_kv_append_attn_run_ragged(ellm_kv_cache* cache, size_t layer, ellm_attn* attn,
                                   const uint32_t* positions, size_t max_position, size_t batch_size,
                                   const void* k_src, const void* v_src, const void* rope,
                                   size_t rope_positions, float eps, void* stream);

/* ------------------------------------------------------------------------ *
 * Position / chunk schedule and a recorded single-token step.
 * ------------------------------------------------------------------------ */

/* One run of every operator of the graph: positions
 * [position_index, position_index + position_interval). */
typedef struct ellm_call {
  size_t position_index;
  size_t position_interval;
} ellm_call;

/*
 * The calls for one request: the prompt [prompt_begin, prompt_end) in chunks of
 * `chunk` positions with a shorter last chunk, then one position at a time up
 * to generation_end (exclusive).  Restates the loop of the reference's serving
 * thread, src/serving/start copy.rs:71-113 (last chunk at
 * prompt_end - (remainder ? remainder : chunk)), without its repetition of the
 * last chunk.  Writes at most `capacity` calls; *n_calls receives the number
 * the schedule has (ELLM_ERR_OUT_OF_RANGE when it exceeds capacity).
 */
int ellm_schedule_calls(size_t prompt_begin, size_t prompt_end, size_t chunk, size_t generation_end,
                        ellm_call* calls, size_t capacity, size_t* n_calls);

/*
 * A recorded sequence of launches (a HIP graph), for the single-token loop in
 * which the host would otherwise issue two launches per layer per token: the
 * reference runs its operator queue once per token behind a spin barrier
 * (src/serving/start.rs:59-77).  Between begin and end, calls of
 * ellm_kv_append_norm_rope / ellm_kv_append / ellm_attn_run_ragged /
 * ellm_positions_advance on `stream` are recorded instead of executed; the
 * per-sequence positions live in device memory, so one recording serves every
 * step.  `stream` must be a created stream, not the null stream.  A handle
 * recorded into a graph must outlive it, and a graph holding a handle's launches
 * must not run at the same time as another launch of that handle (one in flight).
 */
typedef struct ellm_graph ellm_graph;
int ellm_graph_begin(void* stream);
int ellm_graph_end(void* stream, ellm_graph** out_graph);
int ellm_graph_launch(ellm_graph* graph, void* stream);
int ellm_graph_destroy(ellm_graph* graph);

/*
 * A second stream for launches that may run beside those on the caller's stream.
 * A mixed step holds two independent halves, the chunk of a prompt (MFMA-bound) and
 * one new token of the other sequences (HBM-bound); issued one after the other on
 * one stream each waits for the other's last workgroups, side by side they fill
 * each other's tails (16384-token chunk + 32 sequences of 1k-128k cached tokens,
 * one layer: 3.05 -> 2.89 ms).  The reference has no counterpart: its operators
 * run one after another, every thread on each (src/serving/start.rs:59-77).
 *     ellm_side_stream_fork(s, stream);     the side stream waits for what `stream` holds so far
 *     ... launches with ellm_side_stream_get(s) as their stream ...
 *     ... launches on `stream` ...
 *     ellm_side_stream_join(s, stream);     `stream` waits for what the side stream holds so far
 * Works under ellm_graph_begin / ellm_graph_end too (the side stream's launches
 * become a parallel branch of the graph; join before ellm_graph_end).  The two
 * halves must use different handles and write different memory (a handle has one
 * call in flight), and a fork must be joined before the next fork.  The stream has
 * the default priority; destroy waits for its work.
 */
typedef struct ellm_side_stream ellm_side_stream;
int ellm_side_stream_create(ellm_side_stream** out_side);
void* ellm_side_stream_get(ellm_side_stream* side);
int ellm_side_stream_fork(ellm_side_stream* side, void* stream);
int ellm_side_stream_join(ellm_side_stream* side, void* stream);
int ellm_side_stream_destroy(ellm_side_stream* side);

/* positions[i] += by for i < batch_size (device array), in stream order. */
int ellm_positions_advance(uint32_t* positions, size_t batch_size, uint32_t by, void* stream);

/* ------------------------------------------------------------------------ *
 * Projections either side of the attention operator.
 * ------------------------------------------------------------------------ */

/*
 * Fused Q/K/V projection: replaces MatMul3::new / run
 * (src/compiler/mul/matmul3.rs:63-120, 289-385; built by Tensor::matmul3,
 * src/ptensor/tensor.rs:439-498; used by src/qwen3_moe/attention.rs:121-136).
 *     [Cq | Ck | Cv] = hidden . [Wq; Wk; Wv]^T          (binary32 accumulation)
 * Weights are row-major [N][hidden_size] ("W_nt", matmul3.rs:21-29).  Every
 * finished 128-wide head row of Cq and Ck is RMS-normalised (weight 1, eps
 * added to the root mean square) and rotated with a rotary row, as the
 * reference's finalize does (matmul3.rs:243-254, 436-451;
 * src/kernel/x86_64/f16_512/matmul_rms_complex.rs:76-96); arithmetic is
 * binary32 from the sums to the single rounding to the storage type.
 * Row r of `hidden` is token r / batch_size (capacity) of sequence
 * r % batch_size, at position position_index + token (or positions[sequence] +
 * token).  Query rows go to q_state in the same row order; key and value rows go
 * to  state + sequence * kv_strides[0] + head * kv_strides[1] + position *
 * kv_strides[2], which covers both the reference's own k_state layout
 * [position][sequence][kv_head][128] (strides {H*128, 128, B*H*128, 1}, the
 * permuted view of src/qwen3_moe/attention.rs:152-166) and the dimension-first
 * cache of ellm_kv_layer.
 * The rotary row of head h at position p starts at
 *     rope + p * rope_position_stride + h * rope_head_stride    (elements);
 * the reference indexes the table by output column only
 * (rope_base.add(head_col0), matmul3.rs:243-251: position stride 0, head stride
 * 128), a rotary table proper has position stride 128 and head stride 0.
 * Unlike the reference's run, which takes M = batch_size rows and ignores
 * position_interval (matmul3.rs:296-306), all position_interval token rows are
 * projected.
 */
typedef struct ellm_matmul3_desc {
  const void* hidden;   /* device, [max_position_interval][batch_size][hidden_size] */
  const void* q_weight; /* device, [attention_head_num * 128][hidden_size] */
  const void* k_weight; /* device, [kv_head_num * 128][hidden_size] */
  const void* v_weight; /* device, [kv_head_num * 128][hidden_size] */
  void* q_state;        /* device, [max_position_interval][batch_size][attention_head_num][128] */
  void* k_state;        /* device, addressed through kv_strides */
  void* v_state;
  const void* rope;     /* device, (cos, sin) interleaved */
  size_t rope_position_stride; /* elements, multiple of 4 */
  size_t rope_head_stride;     /* elements, multiple of 4 */
  size_t rope_elems;           /* elements in the table (bounds) */
  size_t hidden_size;          /* K: multiple of 64 */
  size_t batch_size;           /* sequence capacity of a token row */
  size_t attention_head_num;
  size_t kv_head_num;
  size_t head_size;            /* 128 */
  size_t kv_strides[4];        /* elements: sequence, kv head, position, 1 */
  size_t sequence_capacity;    /* positions per K/V plane */
  size_t max_position_interval;
  float eps;                   /* the reference passes 1e-6 */
  int dtype;
} ellm_matmul3_desc;
typedef struct ellm_matmul3 ellm_matmul3;
int ellm_matmul3_create(const ellm_matmul3_desc* desc, ellm_matmul3** out_handle);
/* The same on a cache layer with per-sequence capacities (ellm_kv_layer_ragged): key and value
 * rows of sequence i go to state + seq_offsets[i] + head * kv_strides[1] + position *
 * kv_strides[2]; desc->kv_strides[0] and desc->sequence_capacity are ignored. */
int ellm_matmul3_create_ragged(const ellm_matmul3_desc* desc, const ellm_kv_seq_table* table,
                               ellm_matmul3** out_handle);
/* MatMul3::run(position_index, position_interval, batch_size, cpu_num, thread_id) */
int ellm_matmul3_run(ellm_matmul3* handle, size_t position_index, size_t position_interval,
                     size_t batch_size, void* stream);
/* One token per sequence at positions[sequence] (device uint32, clamped to max_position). */
int ellm_matmul3_run_ragged(ellm_matmul3* handle, const uint32_t* positions, size_t max_position,
                            size_t batch_size, void* stream);
int ellm_matmul3_destroy(ellm_matmul3* handle);
/* As ellm_attn_reset, for the counters of the few-rows kernel. */
int ellm_matmul3_reset(ellm_matmul3* handle, void* stream);

/*
 * A single-token step's MatMul3::run followed by Attention::run (position_interval 1) as one
 * call: the two consecutive operators of a layer in the reference's queue
 * (src/qwen3_moe/attention.rs:126-140 then :169-174; run one after the other by
 * src/serving/start.rs:69-73).  After the call q_state, k_state / v_state (the cache rows at
 * the sequences' positions) and the attention output hold what ellm_matmul3_run[_ragged]
 * followed by ellm_attn_run[_ragged] leaves there, to the same tolerances; in between
 * nothing is promised (the projection's launch leaves raw binary32 sums in its handle's
 * workspace and the attention launch normalises and rotates the query and key rows while it
 * loads them, which spares the projection an exchange between its workgroups).  Two
 * launches on `stream`, no allocation, no synchronisation: may be recorded into a graph.
 * The handles must describe the same step: proj's q_state / k_state / v_state are attn's
 * q / k / v, same dtype, head counts, batch_size, kv_strides, sequence_capacity and (for caches
 * with per-sequence capacities) the same sequence table; else ELLM_ERR_INVALID_ARGUMENT.
 * Shapes the fused form does not take (more than 64 sequences, hidden_size not a multiple of
 * 256 or below 1024) run the two ordinary calls: same results.  ellm_matmul3_attn_path tells
 * which (1 fused, 0 two ordinary calls, negative: a status).  Neither handle may have
 * another call in flight.
 */
int ellm_matmul3_attn_run(ellm_matmul3* proj, ellm_attn* attn, size_t position_index,
                          size_t batch_size, void* stream);
/* The same with one position per sequence (device uint32, clamped to max_position). */
int ellm_matmul3_attn_run_ragged(ellm_matmul3* proj, ellm_attn* attn, const uint32_t* positions,
                                 size_t max_position, size_t batch_size, void* stream);
int ellm_matmul3_attn_path(const ellm_matmul3* proj, const ellm_attn* attn, size_t batch_size);

/*
 * Output projection with residual: replaces MatMulAdd::new / run
 * (src/compiler/mul/matmul_add.rs:45-75, 128-232; built by Tensor::matmul_add,
 * src/ptensor/tensor.rs:402-437; used by src/qwen3_moe/attention.rs:176-196 on
 * the [token][sequence][heads * 128] view of the attention output).
 *     output = residual + a . b_nt^T     (binary32, rounded once)
 * a: [max_position_interval][batch_size][k]; b_nt: [n][k]; residual, output:
 * [max_position_interval][batch_size][n]; output may alias residual.
 */
typedef struct ellm_matmul_add_desc {
  const void* a;
  const void* b_nt;
  const void* residual;
  void* output;
  size_t batch_size; /* m_max: sequence capacity of a token row */
  size_t n;          /* multiple of 128 */
  size_t k;          /* multiple of 64 */
  size_t max_position_interval;
  int dtype;
} ellm_matmul_add_desc;
typedef struct ellm_matmul_add ellm_matmul_add;
int ellm_matmul_add_create(const ellm_matmul_add_desc* desc, ellm_matmul_add** out_handle);
/* MatMulAdd::run(position_index, position_interval, batch_size, cpu_num, thread_id) */
int ellm_matmul_add_run(ellm_matmul_add* handle, size_t position_index, size_t position_interval,
                        size_t batch_size, void* stream);
int ellm_matmul_add_destroy(ellm_matmul_add* handle);
int ellm_matmul_add_reset(ellm_matmul_add* handle, void* stream);

/*
 * Which projection kernel and tile shape a call with `rows` activation rows
 * ((position_interval - 1) * batch capacity + batch_size), `heads` output column groups
 * of 128 (attention_head_num + 2 * kv_head_num, or n / 128) and inner size k runs on the
 * current device: 0 = the weight-streaming kernel for at most 64 rows, 1 = MFMA tiles of
 * 128 tokens x one head, 2 = tiles of 256 tokens x one head, 3 = tiles of 256 tokens x two
 * heads; -1 for sizes no handle accepts.  No
 * counterpart in the reference (its MatMul3::run has one code path); it lets a test or a
 * harness see that its shapes reach every kernel.
 */
int ellm_projection_path(size_t rows, size_t heads, size_t k);

#ifdef __cplusplus
}
#endif
#endif /* ELLM_ATTN_H_ */
