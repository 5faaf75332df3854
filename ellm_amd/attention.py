"""Host-side mirror of the reference's attention operator over the C ABI.

``Attention`` takes the argument list of ``Attention::new`` and exposes ``run``
with the meaning of ``Attention::run`` (reference:
src/compiler/mul/attention.rs:41-67 and 69-76).  The reference's ``cpu_num`` /
``thread_id`` pair is accepted and follows its calling convention — every
worker thread calls ``run`` and then meets a barrier (src/serving/start.rs:69-73)
— by letting thread 0 enqueue the launch and every other thread return at once.

Tensors are torch CUDA tensors used as plain device buffers; nothing here
computes with torch.
"""
import ctypes

from . import _lib
from ._lib import AttnDesc, KvDesc, KvRaggedDesc, KvSeqTable, check, load_library


def _dtype_code(t, allow_f32=False):
    import torch

    if t.dtype == torch.float16:
        return _lib.DTYPE_F16
    if t.dtype == torch.bfloat16:
        return _lib.DTYPE_BF16
    if allow_f32 and t.dtype == torch.float32:
        return _lib.DTYPE_F32
    raise TypeError(f"unsupported storage type {t.dtype}")


def _stream_ptr(stream):
    import torch

    if stream is None:
        stream = torch.cuda.current_stream()
    return ctypes.c_void_p(stream.cuda_stream)


def _device_buffer(name, t, need_elems=None, dtype=None):
    """The library is handed raw addresses: make sure `t` is device memory of the stated
    type that holds, from its first element on, the `need_elems` elements the operator
    addresses.  A host address or a short buffer would be a device memory fault."""
    if not getattr(t, "is_cuda", False):
        raise TypeError(f"{name} must be a device (CUDA/HIP) tensor, got {getattr(t, 'device', type(t))}")
    if dtype is not None and t.dtype != dtype:
        raise TypeError(f"{name} is {t.dtype}, expected {dtype}")
    if need_elems is not None:
        have = t.untyped_storage().nbytes() // t.element_size() - t.storage_offset()
        if have < need_elems:
            raise ValueError(f"{name} holds {have} elements from its first one; "
                             f"the operator addresses {need_elems}")
    return t.data_ptr()


def _positions_ptr(positions, batch_size):
    import torch

    if positions.dtype not in (torch.int32, torch.uint32):
        raise TypeError(f"positions must be 32-bit integers, got {positions.dtype}")
    return ctypes.c_void_p(_device_buffer("positions", positions, batch_size))


class Attention:
    """Attention::new / run over device buffers.

    q, out: [max_position_interval, batch_capacity, attention_head_num, head_size]
    k, v:   any 4-d view [sequence, kv_head, position, head_size] (strides are passed on)
    float16 / bfloat16 tensors with head_size 128 run the MFMA kernels; other head sizes up to
    256 and float32 tensors run the library's plain kernel (same arguments and results).
    """

    def __init__(self, q, k, v, out, batch_size, attention_head_num, kv_head_num, head_size,
                 kv_strides, inverse_sqrt_head, lse=None, sequence_capacity=None,
                 max_position_interval=None, seq_table=None):
        """seq_table: a KVCache.layer_ragged(...) view, for a cache whose sequences have different
        capacities (then kv_strides[0] and sequence_capacity are not used)."""
        import torch

        self._lib = load_library()
        self._keep = (q, k, v, out, lse, seq_table)
        interval = int(max_position_interval if max_position_interval is not None else q.shape[0])
        rows = interval * batch_size * attention_head_num
        if seq_table is not None:
            cap = max(seq_table.capacities[:batch_size])
            kv_span = seq_table.span_elems(batch_size, kv_head_num, int(kv_strides[1]))
        else:
            cap = int(sequence_capacity if sequence_capacity is not None else k.shape[2])
            kv_span = ((batch_size - 1) * int(kv_strides[0]) + (kv_head_num - 1) * int(kv_strides[1])
                       + (cap - 1) * int(kv_strides[2]) + head_size)
        d = AttnDesc()
        d.q = _device_buffer("q", q, rows * head_size)
        d.out = _device_buffer("out", out, rows * head_size, q.dtype)
        d.k = _device_buffer("k", k, kv_span, q.dtype)
        d.v = _device_buffer("v", v, kv_span, q.dtype)
        d.lse = _device_buffer("lse", lse, rows, torch.float32) if lse is not None else None
        d.batch_size = batch_size
        d.attention_head_num = attention_head_num
        d.kv_head_num = kv_head_num
        d.head_size = head_size
        for i in range(4):
            d.kv_strides[i] = int(kv_strides[i])
        d.inverse_sqrt_head = float(inverse_sqrt_head)
        d.dtype = _dtype_code(q, allow_f32=True)
        d.sequence_capacity = cap
        d.max_position_interval = interval
        self.desc = d
        self._handle = ctypes.c_void_p()
        if seq_table is not None:
            check(self._lib.ellm_attn_create_ragged(ctypes.byref(d), ctypes.byref(seq_table.table),
                                                    ctypes.byref(self._handle)))
        else:
            check(self._lib.ellm_attn_create(ctypes.byref(d), ctypes.byref(self._handle)))

    @classmethod
    def new(cls, *args, **kwargs):
        return cls(*args, **kwargs)

    def run(self, position_index, position_interval, batch_size, cpu_num=1, thread_id=0,
            stream=None):
        if thread_id != 0:
            return  # the launch is enqueued once, by thread 0
        check(self._lib.ellm_attn_run(self._handle, position_index, position_interval, batch_size,
                                      _stream_ptr(stream)))

    def run_ragged(self, positions, max_position, batch_size, stream=None):
        """Single-token step; positions: uint32/int32 device tensor, one entry per sequence."""
        check(self._lib.ellm_attn_run_ragged(self._handle, _positions_ptr(positions, batch_size),
                                             int(max_position), batch_size, _stream_ptr(stream)))

    def ragged_path(self, max_position, batch_size):
        """Which kernel run_ragged takes for this call: 0 = every plane split alike, 1 = the keys
        of all planes dealt evenly to the workgroups (ellm_attn_ragged_path)."""
        path = self._lib.ellm_attn_ragged_path(self._handle, int(max_position), batch_size)
        if path < 0:
            check(-path)
        return path

    def run_noalloc(self, position, batch_size, positions=None, stream=None):
        """The single-token step through ellm_attn_run_noalloc: this operator's description,
        the library's static device scratch instead of the handle's workspace."""
        pos_ptr = _positions_ptr(positions, batch_size) if positions is not None else None
        check(self._lib.ellm_attn_run_noalloc(ctypes.byref(self.desc), pos_ptr, int(position),
                                              batch_size, _stream_ptr(stream)))

    def reset(self, stream=None):
        """Arrival counters back to zero (after a launch of this handle that did not finish)."""
        check(self._lib.ellm_attn_reset(self._handle, _stream_ptr(stream)))

    def close(self):
        if self._handle:
            check(self._lib.ellm_attn_destroy(self._handle))
            self._handle = ctypes.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class RaggedLayerView:
    """One layer of a cache with per-sequence capacities, from sequence `first_sequence` on:
    base addresses, strides and the sequence table to hand to Attention / MatMul3."""

    def __init__(self, cache, k, v, strides, table, first_sequence):
        self.cache, self.k, self.v, self.strides, self.table = cache, k, v, strides, table
        self.first_sequence = first_sequence
        self.capacities = [int(table.seq_capacity_host[i]) for i in range(table.sequences)]
        self.offsets = cache.offsets[first_sequence:]

    def span_elems(self, batch_size, kv_head_num, head_stride):
        """Elements from the layer base that the first batch_size sequences' planes reach."""
        return max(self.offsets[i] + (kv_head_num - 1) * head_stride + self.capacities[i] * 128
                   for i in range(batch_size))


class KVCache:
    """Keys and values of every layer in one allocation each: [layer][sequence][kv_head]
    [position][128] with one capacity, or (KVCache.ragged) [layer][kv_head][sequence: its own
    positions][128] with a capacity per sequence."""

    def __init__(self, layers, sequences, kv_head_num, capacity, dtype_code, head_size=128,
                 capacities=None):
        self._lib = load_library()
        self._handle = ctypes.c_void_p()
        self.capacities = None
        if capacities is None:
            d = KvDesc(layers, sequences, kv_head_num, head_size, capacity, dtype_code)
            self.desc = d
            check(self._lib.ellm_kv_create(ctypes.byref(d), ctypes.byref(self._handle)))
            return
        caps = (ctypes.c_size_t * len(capacities))(*[int(c) for c in capacities])
        rd = KvRaggedDesc(layers, len(capacities), kv_head_num, head_size, caps, dtype_code)
        self.desc = KvDesc(layers, len(capacities), kv_head_num, head_size, max(capacities), dtype_code)
        self.capacities = [int(c) for c in capacities]
        self.offsets = [128 * sum(self.capacities[:i]) for i in range(len(capacities))]
        self.layer_elems = 128 * sum(self.capacities) * kv_head_num
        check(self._lib.ellm_kv_create_ragged(ctypes.byref(rd), ctypes.byref(self._handle)))

    @classmethod
    def ragged(cls, layers, capacities, kv_head_num, dtype_code, head_size=128):
        return cls(layers, len(capacities), kv_head_num, 0, dtype_code, head_size, capacities=capacities)

    def layer_ragged(self, layer, first_sequence=0):
        k, v = ctypes.c_void_p(), ctypes.c_void_p()
        strides = (ctypes.c_size_t * 4)()
        table = KvSeqTable()
        check(self._lib.ellm_kv_layer_ragged(self._handle, layer, first_sequence, ctypes.byref(k),
                                             ctypes.byref(v), ctypes.byref(strides), ctypes.byref(table)))
        return RaggedLayerView(self, k.value, v.value, list(strides), table, first_sequence)

    def layer_flat_tensors(self, layer, torch_dtype):
        """One layer's K and V of a cache with per-sequence capacities as flat torch tensors
        [kv_head, positions of all sequences, 128]."""
        import torch

        view = self.layer_ragged(layer)
        total = sum(self.capacities)
        shape = (self.desc.kv_head_num, total, self.desc.head_size)

        def wrap(ptr):
            iface = {"shape": (self.layer_elems,), "typestr": "<i2", "data": (ptr, False), "version": 2}
            holder = type("DevBuf", (), {"__cuda_array_interface__": iface})()
            return torch.as_tensor(holder, device="cuda").view(torch_dtype).view(shape)

        return wrap(view.k), wrap(view.v)

    def layer(self, layer):
        k, v = ctypes.c_void_p(), ctypes.c_void_p()
        strides = (ctypes.c_size_t * 4)()
        check(self._lib.ellm_kv_layer(self._handle, layer, ctypes.byref(k), ctypes.byref(v),
                                      ctypes.byref(strides)))
        return k.value, v.value, list(strides)

    def layer_tensors(self, layer, torch_dtype):
        """Borrow one layer's K and V as torch tensors [sequence, kv_head, position, 128]."""
        import torch

        k, v, _ = self.layer(layer)
        d = self.desc
        shape = (d.sequences, d.kv_head_num, d.capacity, d.head_size)
        n = d.sequences * d.kv_head_num * d.capacity * d.head_size

        def wrap(ptr):
            iface = {"shape": (n,), "typestr": "<i2", "data": (ptr, False), "version": 2}
            holder = type("DevBuf", (), {"__cuda_array_interface__": iface})()
            return torch.as_tensor(holder, device="cuda").view(torch_dtype).view(shape)

        return wrap(k), wrap(v)

    def append(self, layer, position_index, k_src, v_src, batch_size=None, stream=None):
        """k_src / v_src: [n_tokens, src_batch_pitch, kv_head, 128] device tensors."""
        n_tokens, pitch = k_src.shape[0], k_src.shape[1]
        if batch_size is None:
            batch_size = pitch
        need = n_tokens * pitch * self.desc.kv_head_num * self.desc.head_size
        check(self._lib.ellm_kv_append(self._handle, layer, position_index, n_tokens, batch_size,
                                       ctypes.c_void_p(_device_buffer("k_src", k_src, need)),
                                       ctypes.c_void_p(_device_buffer("v_src", v_src, need, k_src.dtype)),
                                       pitch, _stream_ptr(stream)))

    def append_norm_rope(self, layer, position_index, k_src, v_src, rope, eps=1e-6, batch_size=None,
                         positions=None, max_position=0, stream=None):
        """append() with the key rows RMS-normalised and rotated by the rotary-table row of
        their position (rope: [positions, 128] device tensor, (cos, sin) interleaved).
        positions: optional uint32/int32 device tensor of per-sequence start positions,
        bounded by max_position."""
        n_tokens, pitch = k_src.shape[0], k_src.shape[1]
        if batch_size is None:
            batch_size = pitch
        pos_ptr = _positions_ptr(positions, batch_size) if positions is not None else None
        need = n_tokens * pitch * self.desc.kv_head_num * self.desc.head_size
        check(self._lib.ellm_kv_append_norm_rope(
            self._handle, layer, position_index, n_tokens, batch_size,
            ctypes.c_void_p(_device_buffer("k_src", k_src, need)),
            ctypes.c_void_p(_device_buffer("v_src", v_src, need, k_src.dtype)), pitch,
            ctypes.c_void_p(_device_buffer("rope", rope, rope.shape[0] * 128, k_src.dtype)),
            rope.shape[0], ctypes.c_float(eps), pos_ptr, int(max_position), _stream_ptr(stream)))

    def append_norm_rope_with_attention(self, layer, attention, position_index, k_src, v_src, rope, eps=1e-6,
                                        batch_size=None, positions=None, max_position=0, stream=None):
        """append_norm_rope() of one new token per sequence and `attention`'s single-token run over
        the cache including it, as one launch (ellm_kv_append_attn_run / _run_ragged).  `attention`
        must have been created over this layer of this cache; k_src, v_src: [1, batch, kv_heads, 128]."""
        if k_src.shape[0] != 1:
            raise ValueError("one new token per sequence")
        pitch = k_src.shape[1]
        if batch_size is None:
            batch_size = pitch
        if batch_size > pitch:
            raise ValueError(f"batch_size {batch_size} exceeds the {pitch} rows of k_src")
        need = pitch * self.desc.kv_head_num * self.desc.head_size
        ks = ctypes.c_void_p(_device_buffer("k_src", k_src, need))
        vs = ctypes.c_void_p(_device_buffer("v_src", v_src, need, k_src.dtype))
        rp = ctypes.c_void_p(_device_buffer("rope", rope, rope.shape[0] * 128, k_src.dtype))
        if positions is None:
            check(self._lib.ellm_kv_append_attn_run(self._handle, layer, attention._handle, position_index, batch_size,
                                                    ks, vs, rp, rope.shape[0], ctypes.c_float(eps), _stream_ptr(stream)))
        else:
            check(self._lib.ellm_kv_append_attn_run_ragged(
                self._handle, layer, attention._handle, _positions_ptr(positions, batch_size), int(max_position),
                batch_size, ks, vs, rp, rope.shape[0], ctypes.c_float(eps), _stream_ptr(stream)))

    def close(self):
        if self._handle:
            check(self._lib.ellm_kv_destroy(self._handle))
            self._handle = ctypes.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
