"""Host-side mirrors of the reference's projection operators either side of attention:
``MatMul3`` (fused Q/K/V projection with RMS norm + rotary rotation of the query and
key heads, src/compiler/mul/matmul3.rs) and ``MatMulAdd`` (output projection plus
residual, src/compiler/mul/matmul_add.rs).  torch tensors are device buffers only."""
import ctypes

from ._lib import MatMul3Desc, MatMulAddDesc, check, load_library
from .attention import _device_buffer, _dtype_code, _positions_ptr, _stream_ptr


class MatMul3:
    """MatMul3::new / run over device buffers.

    hidden:  [max_position_interval, batch_capacity, hidden_size]
    weights: [heads * 128, hidden_size] (row-major N x K, as the reference keeps them)
    q_state: [max_position_interval, batch_capacity, attention_head_num, 128]
    k_state, v_state: any buffers addressed by kv_strides = (sequence, kv head, position, 1)
    rope: (cos, sin) interleaved; row of head h at position p starts at
          p * rope_position_stride + h * rope_head_stride elements
    """

    def __init__(self, hidden, q_weight, q_state, k_weight, k_state, v_weight, v_state, rope,
                 head_dim, batch_size, attention_head_num, kv_head_num, kv_strides,
                 sequence_capacity, rope_position_stride=128, rope_head_stride=0, eps=1e-6,
                 max_position_interval=None, seq_table=None):
        """seq_table: a KVCache.layer_ragged(...) view when k_state / v_state are a cache layer
        whose sequences have different capacities."""
        self._lib = load_library()
        self._keep = (hidden, q_weight, q_state, k_weight, k_state, v_weight, v_state, rope, seq_table)
        dt = hidden.dtype
        hidden_size = hidden.shape[-1]
        interval = int(max_position_interval if max_position_interval is not None else hidden.shape[0])
        rows = interval * batch_size
        if seq_table is not None:
            kv_span = seq_table.span_elems(batch_size, kv_head_num, int(kv_strides[1]))
        else:
            kv_span = ((batch_size - 1) * int(kv_strides[0]) + (kv_head_num - 1) * int(kv_strides[1])
                       + (int(sequence_capacity) - 1) * int(kv_strides[2]) + head_dim)
        d = MatMul3Desc()
        d.hidden = _device_buffer("hidden", hidden, rows * hidden_size)
        d.q_weight = _device_buffer("q_weight", q_weight, attention_head_num * head_dim * hidden_size, dt)
        d.k_weight = _device_buffer("k_weight", k_weight, kv_head_num * head_dim * hidden_size, dt)
        d.v_weight = _device_buffer("v_weight", v_weight, kv_head_num * head_dim * hidden_size, dt)
        d.q_state = _device_buffer("q_state", q_state, rows * attention_head_num * head_dim, dt)
        d.k_state = _device_buffer("k_state", k_state, kv_span, dt)
        d.v_state = _device_buffer("v_state", v_state, kv_span, dt)
        d.rope = _device_buffer("rope", rope, rope.numel(), dt)
        d.rope_position_stride, d.rope_head_stride = int(rope_position_stride), int(rope_head_stride)
        d.rope_elems = rope.numel()
        d.hidden_size = hidden_size
        d.batch_size = batch_size
        d.attention_head_num, d.kv_head_num, d.head_size = attention_head_num, kv_head_num, head_dim
        for i in range(4):
            d.kv_strides[i] = int(kv_strides[i])
        d.sequence_capacity = int(sequence_capacity)
        d.max_position_interval = interval
        d.eps = float(eps)
        d.dtype = _dtype_code(hidden)
        self.desc = d
        self._handle = ctypes.c_void_p()
        if seq_table is not None:
            check(self._lib.ellm_matmul3_create_ragged(ctypes.byref(d), ctypes.byref(seq_table.table),
                                                       ctypes.byref(self._handle)))
        else:
            check(self._lib.ellm_matmul3_create(ctypes.byref(d), ctypes.byref(self._handle)))

    @classmethod
    def new(cls, *args, **kwargs):
        return cls(*args, **kwargs)

    def run(self, position_index, position_interval, batch_size, cpu_num=1, thread_id=0,
            stream=None):
        if thread_id != 0:
            return
        check(self._lib.ellm_matmul3_run(self._handle, position_index, position_interval,
                                         batch_size, _stream_ptr(stream)))

    def run_ragged(self, positions, max_position, batch_size, stream=None):
        check(self._lib.ellm_matmul3_run_ragged(self._handle, _positions_ptr(positions, batch_size),
                                                int(max_position), batch_size, _stream_ptr(stream)))

    def run_with_attention(self, attention, position_index, batch_size, positions=None, stream=None):
        """This projection and `attention` (an ellm_amd.Attention over the same q / k / v) for one
        new token per sequence as one call (ellm_matmul3_attn_run / _run_ragged): what run followed
        by attention.run(position, 1, batch) leaves, with the head rows finished by the attention
        launch.  positions: per-sequence device positions, position_index then their upper bound."""
        if positions is None:
            check(self._lib.ellm_matmul3_attn_run(self._handle, attention._handle, int(position_index),
                                                  batch_size, _stream_ptr(stream)))
        else:
            check(self._lib.ellm_matmul3_attn_run_ragged(self._handle, attention._handle,
                                                         _positions_ptr(positions, batch_size),
                                                         int(position_index), batch_size, _stream_ptr(stream)))

    def attention_path(self, attention, batch_size):
        """1: run_with_attention runs fused for this batch size; 0: as the two ordinary calls."""
        rc = self._lib.ellm_matmul3_attn_path(self._handle, attention._handle, batch_size)
        if rc < 0:
            check(-rc)
        return rc

    def close(self):
        if self._handle:
            check(self._lib.ellm_matmul3_destroy(self._handle))
            self._handle = ctypes.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class MatMulAdd:
    """MatMulAdd::new / run: output = residual + a . b_nt^T.

    a: [max_position_interval, batch_capacity, k]; b_nt: [n, k];
    residual, output: [max_position_interval, batch_capacity, n]
    """

    def __init__(self, a, b_nt, residual, output, m_max=None, n_max=None, k_max=None,
                 max_position_interval=None):
        self._lib = load_library()
        self._keep = (a, b_nt, residual, output)
        d = MatMulAddDesc()
        d.batch_size = int(m_max if m_max is not None else a.shape[1])
        d.n = int(n_max if n_max is not None else b_nt.shape[0])
        d.k = int(k_max if k_max is not None else b_nt.shape[1])
        d.max_position_interval = int(
            max_position_interval if max_position_interval is not None else a.shape[0])
        rows = d.max_position_interval * d.batch_size
        d.a = _device_buffer("a", a, rows * d.k)
        d.b_nt = _device_buffer("b_nt", b_nt, d.n * d.k, a.dtype)
        d.residual = _device_buffer("residual", residual, rows * d.n, a.dtype)
        d.output = _device_buffer("output", output, rows * d.n, a.dtype)
        d.dtype = _dtype_code(a)
        self.desc = d
        self._handle = ctypes.c_void_p()
        check(self._lib.ellm_matmul_add_create(ctypes.byref(d), ctypes.byref(self._handle)))

    @classmethod
    def new(cls, *args, **kwargs):
        return cls(*args, **kwargs)

    def run(self, position_index, position_interval, batch_size, cpu_num=1, thread_id=0,
            stream=None):
        if thread_id != 0:
            return
        check(self._lib.ellm_matmul_add_run(self._handle, position_index, position_interval,
                                            batch_size, _stream_ptr(stream)))

    def close(self):
        if self._handle:
            check(self._lib.ellm_matmul_add_destroy(self._handle))
            self._handle = ctypes.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
