//! `extern "C"` bindings to `libellm_attn.so` (include/ellm_attn.h) and operator wrappers
//! that keep the `new` / `run` signatures of eLLM's own operators, so that
//! `src/ptensor/tensor.rs` and `src/compiler/operator.rs` can build and dispatch them as
//! they do today:
//!
//! * `Attention::new / run`  — src/compiler/mul/attention.rs:41-76
//! * `MatMul3::new / run`    — src/compiler/mul/matmul3.rs:63-120, 289-297
//! * `MatMulAdd::new / run`  — src/compiler/mul/matmul_add.rs:45-75, 128-135
//!
//! This crate is shipped as source and is NOT compiled in this repository (no Rust
//! toolchain in its build container).  `tests/test_abi_layout.py` keeps it honest: it
//! parses the `#[repr(C)]` structs and the `extern "C"` block of this file and checks
//! field order, sizes, offsets and the symbol list against a C probe compiled from the
//! header and against the built library.
//!
//! Pointers handed to the wrappers are DEVICE pointers (hipMalloc, or a layer of
//! `KvCache`).  Every function returns a status (0 = ok); the wrappers turn a non-zero
//! status into a panic with the library's message, which is the reference's own failure
//! mode (`panic = "abort"`, Cargo.toml:49).
#![allow(non_camel_case_types)]
#![cfg_attr(feature = "nightly-f16", feature(f16))]

use core::ffi::{c_char, c_int, c_void};
use core::marker::PhantomData;

/// 16-bit storage element: the reference's `f16` on nightly, the same bits as `u16` on stable.
#[cfg(feature = "nightly-f16")]
pub type Half = f16;
#[cfg(not(feature = "nightly-f16"))]
pub type Half = u16;

pub const ELLM_OK: c_int = 0;
pub const ELLM_ERR_INVALID_ARGUMENT: c_int = 1;
pub const ELLM_ERR_UNSUPPORTED: c_int = 2;
pub const ELLM_ERR_OUT_OF_RANGE: c_int = 3;
pub const ELLM_ERR_HIP: c_int = 4;
pub const ELLM_ERR_NO_DEVICE: c_int = 5;

pub const ELLM_DTYPE_F16: c_int = 0;
pub const ELLM_DTYPE_BF16: c_int = 1;
/// Attention only (`ellm_attn_create`): binary32 storage, the plain kernel.
pub const ELLM_DTYPE_F32: c_int = 2;

// ---- descriptors (field for field as in include/ellm_attn.h) ------------------------------

#[repr(C)]
#[derive(Clone, Copy, Debug)]
pub struct ellm_attn_desc {
    pub q: *const c_void,
    pub k: *const c_void,
    pub v: *const c_void,
    pub out: *mut c_void,
    pub lse: *mut f32,
    pub batch_size: usize,
    pub attention_head_num: usize,
    pub kv_head_num: usize,
    pub head_size: usize,
    pub kv_strides: [usize; 4],
    pub inverse_sqrt_head: f32,
    pub dtype: c_int,
    pub sequence_capacity: usize,
    pub max_position_interval: usize,
}

#[repr(C)]
#[derive(Clone, Copy, Debug)]
pub struct ellm_kv_desc {
    pub layers: usize,
    pub sequences: usize,
    pub kv_head_num: usize,
    pub head_size: usize,
    pub capacity: usize,
    pub dtype: c_int,
}

#[repr(C)]
#[derive(Clone, Copy, Debug)]
pub struct ellm_kv_ragged_desc {
    pub layers: usize,
    pub sequences: usize,
    pub kv_head_num: usize,
    pub head_size: usize,
    pub capacities: *const usize,
    pub dtype: c_int,
}

#[repr(C)]
#[derive(Clone, Copy, Debug)]
pub struct ellm_kv_seq_table {
    pub seq_offsets: *const usize,
    pub seq_capacity: *const u32,
    pub seq_capacity_host: *const usize,
    pub sequences: usize,
}

#[repr(C)]
#[derive(Clone, Copy, Debug, Default, PartialEq, Eq)]
pub struct ellm_call {
    pub position_index: usize,
    pub position_interval: usize,
}

#[repr(C)]
#[derive(Clone, Copy, Debug)]
pub struct ellm_matmul3_desc {
    pub hidden: *const c_void,
    pub q_weight: *const c_void,
    pub k_weight: *const c_void,
    pub v_weight: *const c_void,
    pub q_state: *mut c_void,
    pub k_state: *mut c_void,
    pub v_state: *mut c_void,
    pub rope: *const c_void,
    pub rope_position_stride: usize,
    pub rope_head_stride: usize,
    pub rope_elems: usize,
    pub hidden_size: usize,
    pub batch_size: usize,
    pub attention_head_num: usize,
    pub kv_head_num: usize,
    pub head_size: usize,
    pub kv_strides: [usize; 4],
    pub sequence_capacity: usize,
    pub max_position_interval: usize,
    pub eps: f32,
    pub dtype: c_int,
}

#[repr(C)]
#[derive(Clone, Copy, Debug)]
pub struct ellm_matmul_add_desc {
    pub a: *const c_void,
    pub b_nt: *const c_void,
    pub residual: *const c_void,
    pub output: *mut c_void,
    pub batch_size: usize,
    pub n: usize,
    pub k: usize,
    pub max_position_interval: usize,
    pub dtype: c_int,
}

// opaque handles
#[repr(C)]
pub struct ellm_attn {
    _private: [u8; 0],
}
#[repr(C)]
pub struct ellm_kv_cache {
    _private: [u8; 0],
}
#[repr(C)]
pub struct ellm_graph {
    _private: [u8; 0],
}
#[repr(C)]
pub struct ellm_side_stream {
    _private: [u8; 0],
}
#[repr(C)]
pub struct ellm_matmul3 {
    _private: [u8; 0],
}
#[repr(C)]
pub struct ellm_matmul_add {
    _private: [u8; 0],
}

/// A HIP stream (`hipStream_t`); null is the null stream.
pub type Stream = *mut c_void;

extern "C" {
    pub fn ellm_last_error_string() -> *const c_char;
    pub fn ellm_attn_version() -> c_int;
    pub fn ellm_device_count() -> c_int;

    pub fn ellm_attn_create(desc: *const ellm_attn_desc, out_handle: *mut *mut ellm_attn) -> c_int;
    pub fn ellm_attn_create_ragged(
        desc: *const ellm_attn_desc,
        table: *const ellm_kv_seq_table,
        out_handle: *mut *mut ellm_attn,
    ) -> c_int;
    pub fn ellm_attn_destroy(handle: *mut ellm_attn) -> c_int;
    pub fn ellm_attn_reset(handle: *mut ellm_attn, stream: Stream) -> c_int;
    pub fn ellm_matmul3_reset(handle: *mut ellm_matmul3, stream: Stream) -> c_int;
    pub fn ellm_matmul_add_reset(handle: *mut ellm_matmul_add, stream: Stream) -> c_int;
    pub fn ellm_attn_run(
        handle: *mut ellm_attn,
        position_index: usize,
        position_interval: usize,
        batch_size: usize,
        stream: Stream,
    ) -> c_int;
    pub fn ellm_attn_run_ragged(
        handle: *mut ellm_attn,
        positions: *const u32,
        max_position: usize,
        batch_size: usize,
        stream: Stream,
    ) -> c_int;
    pub fn ellm_attn_ragged_path(handle: *const ellm_attn, max_position: usize, batch_size: usize) -> c_int;
    pub fn ellm_attn_run_noalloc(
        desc: *const ellm_attn_desc,
        positions: *const u32,
        position: usize,
        batch_size: usize,
        stream: Stream,
    ) -> c_int;

    pub fn ellm_kv_create(desc: *const ellm_kv_desc, out_cache: *mut *mut ellm_kv_cache) -> c_int;
    pub fn ellm_kv_create_ragged(desc: *const ellm_kv_ragged_desc, out_cache: *mut *mut ellm_kv_cache) -> c_int;
    pub fn ellm_kv_destroy(cache: *mut ellm_kv_cache) -> c_int;
    pub fn ellm_kv_layer(
        cache: *const ellm_kv_cache,
        layer: usize,
        k: *mut *mut c_void,
        v: *mut *mut c_void,
        kv_strides: *mut usize, // [4]
    ) -> c_int;
    pub fn ellm_kv_layer_ragged(
        cache: *const ellm_kv_cache,
        layer: usize,
        first_sequence: usize,
        k: *mut *mut c_void,
        v: *mut *mut c_void,
        kv_strides: *mut usize, // [4]
        table: *mut ellm_kv_seq_table,
    ) -> c_int;
    pub fn ellm_kv_append(
        cache: *mut ellm_kv_cache,
        layer: usize,
        position_index: usize,
        n_tokens: usize,
        batch_size: usize,
        k_src: *const c_void,
        v_src: *const c_void,
        src_batch_pitch: usize,
        stream: Stream,
    ) -> c_int;
    pub fn ellm_kv_append_norm_rope(
        cache: *mut ellm_kv_cache,
        layer: usize,
        position_index: usize,
        n_tokens: usize,
        batch_size: usize,
        k_src: *const c_void,
        v_src: *const c_void,
        src_batch_pitch: usize,
        rope: *const c_void,
        rope_positions: usize,
        eps: f32,
        positions: *const u32,
        max_position: usize,
        stream: Stream,
    ) -> c_int;
    pub fn ellm_kv_append_attn_run(
        cache: *mut ellm_kv_cache,
        layer: usize,
        attn: *mut ellm_attn,
        position_index: usize,
        batch_size: usize,
        k_src: *const c_void,
        v_src: *const c_void,
        rope: *const c_void,
        rope_positions: usize,
        eps: f32,
        stream: Stream,
    ) -> c_int;
    pub fn ellm_kv_append_attn_run_ragged(
        cache: *mut ellm_kv_cache,
        layer: usize,
        attn: *mut ellm_attn,
        positions: *const u32,
        max_position: usize,
        batch_size: usize,
        k_src: *const c_void,
        v_src: *const c_void,
        rope: *const c_void,
        rope_positions: usize,
        eps: f32,
        stream: Stream,
    ) -> c_int;

    pub fn ellm_schedule_calls(
        prompt_begin: usize,
        prompt_end: usize,
        chunk: usize,
        generation_end: usize,
        calls: *mut ellm_call,
        capacity: usize,
        n_calls: *mut usize,
    ) -> c_int;
    pub fn ellm_graph_begin(stream: Stream) -> c_int;
    pub fn ellm_graph_end(stream: Stream, out_graph: *mut *mut ellm_graph) -> c_int;
    pub fn ellm_graph_launch(graph: *mut ellm_graph, stream: Stream) -> c_int;
    pub fn ellm_graph_destroy(graph: *mut ellm_graph) -> c_int;
    pub fn ellm_side_stream_create(out_side: *mut *mut ellm_side_stream) -> c_int;
    pub fn ellm_side_stream_get(side: *mut ellm_side_stream) -> Stream;
    pub fn ellm_side_stream_fork(side: *mut ellm_side_stream, stream: Stream) -> c_int;
    pub fn ellm_side_stream_join(side: *mut ellm_side_stream, stream: Stream) -> c_int;
    pub fn ellm_side_stream_destroy(side: *mut ellm_side_stream) -> c_int;
    pub fn ellm_positions_advance(positions: *mut u32, batch_size: usize, by: u32, stream: Stream) -> c_int;

    pub fn ellm_matmul3_create(desc: *const ellm_matmul3_desc, out_handle: *mut *mut ellm_matmul3) -> c_int;
    pub fn ellm_matmul3_create_ragged(
        desc: *const ellm_matmul3_desc,
        table: *const ellm_kv_seq_table,
        out_handle: *mut *mut ellm_matmul3,
    ) -> c_int;
    pub fn ellm_matmul3_run(
        handle: *mut ellm_matmul3,
        position_index: usize,
        position_interval: usize,
        batch_size: usize,
        stream: Stream,
    ) -> c_int;
    pub fn ellm_matmul3_run_ragged(
        handle: *mut ellm_matmul3,
        positions: *const u32,
        max_position: usize,
        batch_size: usize,
        stream: Stream,
    ) -> c_int;
    pub fn ellm_matmul3_destroy(handle: *mut ellm_matmul3) -> c_int;
    pub fn ellm_matmul3_attn_run(
        proj: *mut ellm_matmul3,
        attn: *mut ellm_attn,
        position_index: usize,
        batch_size: usize,
        stream: Stream,
    ) -> c_int;
    pub fn ellm_matmul3_attn_run_ragged(
        proj: *mut ellm_matmul3,
        attn: *mut ellm_attn,
        positions: *const u32,
        max_position: usize,
        batch_size: usize,
        stream: Stream,
    ) -> c_int;
    pub fn ellm_matmul3_attn_path(proj: *const ellm_matmul3, attn: *const ellm_attn, batch_size: usize) -> c_int;

    pub fn ellm_matmul_add_create(desc: *const ellm_matmul_add_desc, out_handle: *mut *mut ellm_matmul_add) -> c_int;
    pub fn ellm_matmul_add_run(
        handle: *mut ellm_matmul_add,
        position_index: usize,
        position_interval: usize,
        batch_size: usize,
        stream: Stream,
    ) -> c_int;
    pub fn ellm_matmul_add_destroy(handle: *mut ellm_matmul_add) -> c_int;

    pub fn ellm_projection_path(rows: usize, heads: usize, k: usize) -> c_int;
}

// ---- safe-ish wrappers with the reference's signatures ----------------------------------------

fn check(status: c_int, what: &str) {
    if status != ELLM_OK {
        let msg = unsafe {
            let p = ellm_last_error_string();
            if p.is_null() {
                String::new()
            } else {
                std::ffi::CStr::from_ptr(p).to_string_lossy().into_owned()
            }
        };
        panic!("{what}: ellm status {status}: {msg}");
    }
}

/// What the GPU path needs beyond the reference's argument lists and cannot derive from
/// them: the stream to launch on, the storage type, and the capacities that size the
/// launches (the reference's operators never check a position against anything).
#[derive(Clone, Copy, Debug)]
pub struct Placement {
    pub stream: Stream,
    pub dtype: c_int,
    /// positions per K/V plane
    pub sequence_capacity: usize,
    /// largest `position_interval` a `run` will be given (the chunk size; 1 for a decode-only graph)
    pub max_position_interval: usize,
}

/// `compiler::mul::attention::Attention<T>` (src/compiler/mul/attention.rs:12-27).
pub struct Attention<T> {
    handle: *mut ellm_attn,
    stream: Stream,
    _t: PhantomData<T>,
}
// the reference marks its operators Send + Sync (src/compiler/operator.rs:253-254); a handle
// may be used from one thread at a time, which run()'s thread_id == 0 rule guarantees
unsafe impl<T> Send for Attention<T> {}
unsafe impl<T> Sync for Attention<T> {}

impl Attention<Half> {
    /// The argument list of `Attention::new` (attention.rs:41-54) followed by the placement.
    /// `batch_size` is the capacity in sequences (the Q/O row pitch), `kv_strides` the four
    /// element strides of the K/V view `[sequence][kv_head][position][head_size]`;
    /// `kv_head_num` is the number of KV heads (`k_tensor.shape[1]` of that view —
    /// `Tensor::attention` passes `shape[2]` today, src/ptensor/tensor.rs:131, which is the
    /// sequence length: that call site has to change).
    #[allow(clippy::too_many_arguments)]
    pub fn new(
        q_ptr: *const Half,
        k_ptr: *const Half,
        v_ptr: *const Half,
        output_ptr: *mut Half,
        batch_size: usize,
        attention_head_num: usize,
        kv_head_num: usize,
        head_size: usize,
        kv_strides: Vec<usize>,
        inverse_sqrt_head: f32,
        place: Placement,
    ) -> Self {
        assert_eq!(kv_strides.len(), 4, "kv_strides: [sequence, kv_head, position, element]");
        let desc = ellm_attn_desc {
            q: q_ptr.cast(),
            k: k_ptr.cast(),
            v: v_ptr.cast(),
            out: output_ptr.cast(),
            lse: core::ptr::null_mut(),
            batch_size,
            attention_head_num,
            kv_head_num,
            head_size,
            kv_strides: [kv_strides[0], kv_strides[1], kv_strides[2], kv_strides[3]],
            inverse_sqrt_head,
            dtype: place.dtype,
            sequence_capacity: place.sequence_capacity,
            max_position_interval: place.max_position_interval,
        };
        let mut handle = core::ptr::null_mut();
        check(unsafe { ellm_attn_create(&desc, &mut handle) }, "ellm_attn_create");
        Self { handle, stream: place.stream, _t: PhantomData }
    }

    /// `Attention::run` (attention.rs:69-76).  Every worker thread of the reference's
    /// runtime calls `run` and then waits at the barrier (src/serving/start.rs:69-73):
    /// thread 0 enqueues the launch, the others return at once; stream order gives what
    /// the barrier gave.
    pub fn run(&self, position_index: usize, position_interval: usize, batch_size: usize, _cpu_num: usize, thread_id: usize) {
        if thread_id != 0 {
            return;
        }
        check(
            unsafe { ellm_attn_run(self.handle, position_index, position_interval, batch_size, self.stream) },
            "ellm_attn_run",
        );
    }

    /// One token per sequence at `positions[sequence]` (device array); no counterpart in the
    /// reference, whose batch shares one position.
    pub fn run_ragged(&self, positions: *const u32, max_position: usize, batch_size: usize) {
        check(
            unsafe { ellm_attn_run_ragged(self.handle, positions, max_position, batch_size, self.stream) },
            "ellm_attn_run_ragged",
        );
    }
}

impl<T> Drop for Attention<T> {
    fn drop(&mut self) {
        unsafe { ellm_attn_destroy(self.handle) };
    }
}

/// `compiler::mul::matmul3::MatMul3<T>` (src/compiler/mul/matmul3.rs:30-58).
pub struct MatMul3<T> {
    handle: *mut ellm_matmul3,
    stream: Stream,
    _t: PhantomData<T>,
}
unsafe impl<T> Send for MatMul3<T> {}
unsafe impl<T> Sync for MatMul3<T> {}

impl MatMul3<Half> {
    /// The argument list of `MatMul3::new` (matmul3.rs:63-82): the five tiling steps are
    /// accepted and ignored (the GPU kernels choose their own tiles), `m_row` is the batch
    /// capacity of a token row, `col` = K, `b_q_row` / `b_kv_row` = Nq / Nkv.  Then what the
    /// GPU path needs in addition: where key / value rows go (`kv_strides` of the state
    /// they are written to) and the rotary table's indexing.
    #[allow(clippy::too_many_arguments)]
    pub fn new(
        hidden_ptr: *const Half,
        q_weight_ptr_nt: *const Half,
        q_state_ptr: *mut Half,
        k_weight_ptr_nt: *const Half,
        k_state_ptr: *mut Half,
        v_weight_ptr_nt: *const Half,
        v_state_ptr: *mut Half,
        rope_ptr: *const Half,
        head_dim: usize,
        m_row: usize,
        col: usize,
        b_q_row: usize,
        b_kv_row: usize,
        _a_row_step_macro: usize,
        _b_row_step_macro: usize,
        _column_step_macro: usize,
        _a_row_step_micro: usize,
        _b_row_step_micro: usize,
        kv_strides: [usize; 4],
        rope_position_stride: usize,
        rope_head_stride: usize,
        rope_elems: usize,
        place: Placement,
    ) -> Self {
        let desc = ellm_matmul3_desc {
            hidden: hidden_ptr.cast(),
            q_weight: q_weight_ptr_nt.cast(),
            k_weight: k_weight_ptr_nt.cast(),
            v_weight: v_weight_ptr_nt.cast(),
            q_state: q_state_ptr.cast(),
            k_state: k_state_ptr.cast(),
            v_state: v_state_ptr.cast(),
            rope: rope_ptr.cast(),
            rope_position_stride,
            rope_head_stride,
            rope_elems,
            hidden_size: col,
            batch_size: m_row,
            attention_head_num: b_q_row / head_dim,
            kv_head_num: b_kv_row / head_dim,
            head_size: head_dim,
            kv_strides,
            sequence_capacity: place.sequence_capacity,
            max_position_interval: place.max_position_interval,
            eps: 1e-6, // what the reference's finalize passes (matmul3.rs:243-254)
            dtype: place.dtype,
        };
        let mut handle = core::ptr::null_mut();
        check(unsafe { ellm_matmul3_create(&desc, &mut handle) }, "ellm_matmul3_create");
        Self { handle, stream: place.stream, _t: PhantomData }
    }

    /// `MatMul3::run` (matmul3.rs:289-297).
    pub fn run(&self, position_index: usize, position_interval: usize, batch_size: usize, _cpu_num: usize, thread_id: usize) {
        if thread_id != 0 {
            return;
        }
        check(
            unsafe { ellm_matmul3_run(self.handle, position_index, position_interval, batch_size, self.stream) },
            "ellm_matmul3_run",
        );
    }

    pub fn run_ragged(&self, positions: *const u32, max_position: usize, batch_size: usize) {
        check(
            unsafe { ellm_matmul3_run_ragged(self.handle, positions, max_position, batch_size, self.stream) },
            "ellm_matmul3_run_ragged",
        );
    }

    /// This operator and the `Attention` that follows it in the queue
    /// (src/qwen3_moe/attention.rs:126-174) for a step of one position, as one call: what
    /// `run(position_index, 1, ..)` followed by `attention.run(position_index, 1, ..)` leaves.
    pub fn run_with_attention(&self, attention: &Attention<T>, position_index: usize, batch_size: usize, thread_id: usize) {
        if thread_id != 0 {
            return;
        }
        check(
            unsafe { ellm_matmul3_attn_run(self.handle, attention.handle, position_index, batch_size, self.stream) },
            "ellm_matmul3_attn_run",
        );
    }
}

impl<T> Drop for MatMul3<T> {
    fn drop(&mut self) {
        unsafe { ellm_matmul3_destroy(self.handle) };
    }
}

/// The reference's tiling parameters (src/init/matmul_params.rs:1-8); accepted for source
/// compatibility and ignored.
#[derive(Clone, Copy, Debug, Default)]
pub struct MatMulParams {
    pub a_row_step_macro: usize,
    pub b_row_step_macro: usize,
    pub column_step_macro: usize,
    pub a_row_step_micro: usize,
    pub b_row_step_micro: usize,
}

/// `compiler::mul::matmul_add::MatMulAdd<T>` (src/compiler/mul/matmul_add.rs:17-35).
pub struct MatMulAdd<T> {
    handle: *mut ellm_matmul_add,
    stream: Stream,
    _t: PhantomData<T>,
}
unsafe impl<T> Send for MatMulAdd<T> {}
unsafe impl<T> Sync for MatMulAdd<T> {}

impl MatMulAdd<Half> {
    /// The argument list of `MatMulAdd::new` (matmul_add.rs:45-54) followed by the placement
    /// (`sequence_capacity` is not used by this operator).
    ///
    /// # Safety
    /// As in the reference, the pointers must stay valid for the operator's lifetime; here
    /// they must be device pointers.
    #[allow(clippy::too_many_arguments)]
    pub unsafe fn new(
        ptr1: *const Half,
        ptr2_b_nt_nxk: *const Half,
        ptr3_residual: *const Half,
        output_ptr: *mut Half,
        _params: MatMulParams,
        m_max: usize,
        n_max: usize,
        k_max: usize,
        place: Placement,
    ) -> Self {
        let desc = ellm_matmul_add_desc {
            a: ptr1.cast(),
            b_nt: ptr2_b_nt_nxk.cast(),
            residual: ptr3_residual.cast(),
            output: output_ptr.cast(),
            batch_size: m_max,
            n: n_max,
            k: k_max,
            max_position_interval: place.max_position_interval,
            dtype: place.dtype,
        };
        let mut handle = core::ptr::null_mut();
        check(ellm_matmul_add_create(&desc, &mut handle), "ellm_matmul_add_create");
        Self { handle, stream: place.stream, _t: PhantomData }
    }

    /// `MatMulAdd::run` (matmul_add.rs:128-135).
    pub fn run(&self, position_index: usize, position_interval: usize, batch_size: usize, _cpu_num: usize, thread_id: usize) {
        if thread_id != 0 {
            return;
        }
        check(
            unsafe { ellm_matmul_add_run(self.handle, position_index, position_interval, batch_size, self.stream) },
            "ellm_matmul_add_run",
        );
    }
}

impl<T> Drop for MatMulAdd<T> {
    fn drop(&mut self) {
        unsafe { ellm_matmul_add_destroy(self.handle) };
    }
}

/// The per-layer K/V buffers of `memory::Cache` (src/memory/cache.rs:23, 69-75) as one
/// device allocation each for keys and values, written in place at token coordinates.
pub struct KvCache {
    handle: *mut ellm_kv_cache,
}
unsafe impl Send for KvCache {}
unsafe impl Sync for KvCache {}

/// One layer of a cache: device base pointers and the four strides for `Attention::new` /
/// `MatMul3::new`; `table` is set for caches with per-sequence capacities.
#[derive(Clone, Copy, Debug)]
pub struct KvLayer {
    pub k: *mut c_void,
    pub v: *mut c_void,
    pub kv_strides: [usize; 4],
    pub table: Option<ellm_kv_seq_table>,
}

impl KvCache {
    pub fn new(layers: usize, sequences: usize, kv_head_num: usize, head_size: usize, capacity: usize, dtype: c_int) -> Self {
        let desc = ellm_kv_desc { layers, sequences, kv_head_num, head_size, capacity, dtype };
        let mut handle = core::ptr::null_mut();
        check(unsafe { ellm_kv_create(&desc, &mut handle) }, "ellm_kv_create");
        Self { handle }
    }

    /// One capacity per sequence (slot): static, non-paged, contiguous per plane.
    pub fn new_ragged(layers: usize, kv_head_num: usize, head_size: usize, capacities: &[usize], dtype: c_int) -> Self {
        let desc = ellm_kv_ragged_desc {
            layers,
            sequences: capacities.len(),
            kv_head_num,
            head_size,
            capacities: capacities.as_ptr(),
            dtype,
        };
        let mut handle = core::ptr::null_mut();
        check(unsafe { ellm_kv_create_ragged(&desc, &mut handle) }, "ellm_kv_create_ragged");
        Self { handle }
    }

    pub fn layer(&self, layer: usize) -> KvLayer {
        let (mut k, mut v) = (core::ptr::null_mut(), core::ptr::null_mut());
        let mut kv_strides = [0usize; 4];
        check(unsafe { ellm_kv_layer(self.handle, layer, &mut k, &mut v, kv_strides.as_mut_ptr()) }, "ellm_kv_layer");
        KvLayer { k, v, kv_strides, table: None }
    }

    pub fn layer_ragged(&self, layer: usize, first_sequence: usize) -> KvLayer {
        let (mut k, mut v) = (core::ptr::null_mut(), core::ptr::null_mut());
        let mut kv_strides = [0usize; 4];
        let mut table = ellm_kv_seq_table {
            seq_offsets: core::ptr::null(),
            seq_capacity: core::ptr::null(),
            seq_capacity_host: core::ptr::null(),
            sequences: 0,
        };
        check(
            unsafe { ellm_kv_layer_ragged(self.handle, layer, first_sequence, &mut k, &mut v, kv_strides.as_mut_ptr(), &mut table) },
            "ellm_kv_layer_ragged",
        );
        KvLayer { k, v, kv_strides, table: Some(table) }
    }

    pub fn as_ptr(&self) -> *mut ellm_kv_cache {
        self.handle
    }
}

impl Drop for KvCache {
    fn drop(&mut self) {
        unsafe { ellm_kv_destroy(self.handle) };
    }
}

/// The calls of one request: the prompt in chunks, a shorter last chunk, then one position
/// per call (src/serving/start copy.rs:71-113).
pub fn schedule_calls(prompt_begin: usize, prompt_end: usize, chunk: usize, generation_end: usize) -> Vec<ellm_call> {
    let mut n = 0usize;
    // first pass counts (capacity 0 is allowed and reports ELLM_ERR_OUT_OF_RANGE with the count)
    unsafe { ellm_schedule_calls(prompt_begin, prompt_end, chunk, generation_end, core::ptr::null_mut(), 0, &mut n) };
    let mut calls = vec![ellm_call::default(); n];
    check(
        unsafe { ellm_schedule_calls(prompt_begin, prompt_end, chunk, generation_end, calls.as_mut_ptr(), n, &mut n) },
        "ellm_schedule_calls",
    );
    calls
}
