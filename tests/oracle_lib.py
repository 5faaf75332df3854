"""ctypes access to the CPU oracle (oracle/libellm_oracle.so) for the tests.

The oracle is test infrastructure: it restates the reference's attention
arithmetic in binary32 and is only ever used as the checker.
"""
import ctypes
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_DIR = os.path.join(ROOT, "oracle")
ORACLE_SO = os.path.join(ORACLE_DIR, "libellm_oracle.so")

F16, BF16, F32 = 0, 1, 2


class OracleAttn(ctypes.Structure):
    _fields_ = [
        ("q", ctypes.c_void_p),
        ("k", ctypes.c_void_p),
        ("v", ctypes.c_void_p),
        ("out", ctypes.c_void_p),
        ("lse", ctypes.c_void_p),
        ("batch_capacity", ctypes.c_size_t),
        ("attention_head_num", ctypes.c_size_t),
        ("kv_head_num", ctypes.c_size_t),
        ("head_size", ctypes.c_size_t),
        ("kv_strides", ctypes.c_size_t * 4),
        ("inverse_sqrt_head", ctypes.c_float),
        ("dtype", ctypes.c_int),
    ]


_lib = None


def load():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(ORACLE_SO):
        subprocess.check_call(["make", "-C", ORACLE_DIR])
    lib = ctypes.CDLL(ORACLE_SO)
    sz, vp, f = ctypes.c_size_t, ctypes.c_void_p, ctypes.c_float
    lib.ellm_oracle_dot_product_f32.restype = f
    lib.ellm_oracle_dot_product_f32.argtypes = [vp, vp, sz]
    lib.ellm_oracle_scalar_vector_mul_and_acc_f32.restype = None
    lib.ellm_oracle_scalar_vector_mul_and_acc_f32.argtypes = [f, vp, f, vp, sz]
    lib.ellm_oracle_scale_softmax_f32.restype = None
    lib.ellm_oracle_scale_softmax_f32.argtypes = [vp, vp, sz, f]
    lib.ellm_oracle_flash_attention.restype = None
    lib.ellm_oracle_flash_attention.argtypes = [vp, vp, vp, vp, vp, f, sz, sz, sz, ctypes.c_int]
    lib.ellm_oracle_assign.restype = ctypes.c_int
    lib.ellm_oracle_assign.argtypes = [sz, sz, sz, ctypes.POINTER(sz), ctypes.POINTER(sz)]
    lib.ellm_oracle_attention_run.restype = ctypes.c_int
    lib.ellm_oracle_attention_run.argtypes = [ctypes.POINTER(OracleAttn), sz, sz, sz, vp, sz, sz]
    lib.ellm_oracle_attention_run_threads.restype = ctypes.c_double
    lib.ellm_oracle_attention_run_threads.argtypes = [
        ctypes.POINTER(OracleAttn), sz, sz, sz, vp, sz, ctypes.c_int, sz]
    lib.ellm_oracle_attention_rows_threads.restype = ctypes.c_double
    lib.ellm_oracle_attention_rows_threads.argtypes = [
        ctypes.POINTER(OracleAttn), sz, vp, sz, vp, vp, sz]
    lib.ellm_oracle_attention_rows_threads_ex.restype = ctypes.c_double
    lib.ellm_oracle_attention_rows_threads_ex.argtypes = [
        ctypes.POINTER(OracleAttn), sz, vp, vp, sz, vp, vp, sz, ctypes.c_int]
    lib.ellm_oracle_f32_to_f16.restype = ctypes.c_uint16
    lib.ellm_oracle_f32_to_f16.argtypes = [f]
    lib.ellm_oracle_f16_to_f32.restype = f
    lib.ellm_oracle_f16_to_f32.argtypes = [ctypes.c_uint16]
    lib.ellm_oracle_f32_to_bf16.restype = ctypes.c_uint16
    lib.ellm_oracle_f32_to_bf16.argtypes = [f]
    lib.ellm_oracle_bf16_to_f32.restype = f
    lib.ellm_oracle_bf16_to_f32.argtypes = [ctypes.c_uint16]
    lib.ellm_oracle_barrier_selftest.restype = ctypes.c_int
    lib.ellm_oracle_barrier_selftest.argtypes = [sz, sz]
    lib.ellm_oracle_schedule_calls.restype = ctypes.c_long
    lib.ellm_oracle_schedule_calls.argtypes = [sz, sz, sz, sz, vp, vp, sz]
    lib.ellm_oracle_rms_norm_f32.restype = None
    lib.ellm_oracle_rms_norm_f32.argtypes = [vp, vp, sz, f]
    lib.ellm_oracle_complex_mul_f32.restype = None
    lib.ellm_oracle_complex_mul_f32.argtypes = [vp, vp, vp, sz]
    lib.ellm_oracle_norm_rope_row.restype = None
    lib.ellm_oracle_norm_rope_row.argtypes = [vp, vp, vp, sz, f, ctypes.c_int]
    lib.ellm_oracle_kv_append_norm_rope.restype = ctypes.c_int
    lib.ellm_oracle_kv_append_norm_rope.argtypes = [vp, vp, sz, sz, sz, sz, sz, sz, vp, vp, sz, vp,
                                                    sz, f, vp, ctypes.c_int]
    lib.ellm_oracle_matmul_nt.restype = None
    lib.ellm_oracle_matmul_nt.argtypes = [vp, vp, vp, sz, sz, sz, ctypes.c_int]
    lib.ellm_oracle_matmul3.restype = ctypes.c_int
    lib.ellm_oracle_matmul3.argtypes = [vp, vp, vp, vp, vp, vp, vp, vp, sz, sz, sz, sz, sz, sz, sz,
                                        sz, sz, ctypes.POINTER(sz * 4), sz, sz, sz, vp, f,
                                        ctypes.c_int]
    lib.ellm_oracle_matmul_add.restype = None
    lib.ellm_oracle_matmul_add.argtypes = [vp, vp, vp, vp, sz, sz, sz, sz, sz, ctypes.c_int]
    _lib = lib
    return lib


def _ptr(a):
    return ctypes.c_void_p(a.ctypes.data) if a is not None else None


# ---- storage conversions on numpy arrays (bit patterns in uint16) -------------

def to_storage(x32, dtype):
    """binary32 array -> storage array (float16 / uint16 bf16 bits / float32)."""
    x32 = np.ascontiguousarray(x32, dtype=np.float32)
    if dtype == F16:
        return x32.astype(np.float16)
    if dtype == BF16:
        u = x32.view(np.uint32).astype(np.uint64)
        u = (u + 0x7FFF + ((u >> 16) & 1)) >> 16
        return u.astype(np.uint16)
    return x32


def from_storage(a, dtype):
    if dtype == F16:
        return np.asarray(a).view(np.float16).astype(np.float32)
    if dtype == BF16:
        return (np.asarray(a).view(np.uint16).astype(np.uint32) << 16).view(np.float32)
    return np.asarray(a, dtype=np.float32)


def storage_np_dtype(dtype):
    return {F16: np.float16, BF16: np.uint16, F32: np.float32}[dtype]


def schedule_calls(prompt_begin, prompt_end, chunk, generation_end, capacity=None):
    """The oracle's (position_index, position_interval) list, or None when it does not fit."""
    if capacity is None:
        capacity = max(prompt_end - prompt_begin, 0) + max(generation_end - prompt_end, 0) + 2
    pos = np.zeros(max(capacity, 1), dtype=np.uintp)
    itv = np.zeros(max(capacity, 1), dtype=np.uintp)
    n = load().ellm_oracle_schedule_calls(prompt_begin, prompt_end, chunk, generation_end,
                                          _ptr(pos), _ptr(itv), capacity)
    if n < 0:
        return None
    return [(int(pos[i]), int(itv[i])) for i in range(n)]


def rms_norm(x, eps):
    """src/kernel/generic/rms_norm.rs restated; x: float32 vector."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.zeros_like(x)
    load().ellm_oracle_rms_norm_f32(_ptr(x), _ptr(out), x.size, ctypes.c_float(eps))
    return out


def complex_mul(x, y):
    """src/kernel/generic/complex_mul.rs restated; interleaved (re, im) float32 vectors."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    y = np.ascontiguousarray(y, dtype=np.float32)
    out = np.zeros_like(x)
    load().ellm_oracle_complex_mul_f32(_ptr(x), _ptr(y), _ptr(out), x.size)
    return out


def norm_rope_row(row, rope_row, eps, dtype):
    """One stored head row: RMS norm, rotation by one rotary-table row, stored again."""
    out = np.zeros_like(row)
    load().ellm_oracle_norm_rope_row(_ptr(row), _ptr(rope_row), _ptr(out), row.size,
                                     ctypes.c_float(eps), dtype)
    return out


def kv_append_norm_rope(k_cache, v_cache, position_index, k_src, v_src, rope, eps, dtype,
                        batch_size=None, positions=None):
    """k_cache / v_cache: [sequence, kv_head, capacity, D] storage arrays, written in place;
    k_src / v_src: [n_tokens, src_batch_pitch, kv_head, D]; rope: [positions, D].
    Returns the oracle's status (0 ok, 1 a position outside the cache or the table)."""
    _, kv_heads, capacity, d = k_cache.shape
    n_tokens, pitch = k_src.shape[0], k_src.shape[1]
    if batch_size is None:
        batch_size = pitch
    pos = None
    if positions is not None:
        pos = np.ascontiguousarray(positions, dtype=np.uint32)
    return load().ellm_oracle_kv_append_norm_rope(
        _ptr(k_cache), _ptr(v_cache), kv_heads, capacity, d, position_index, n_tokens, batch_size,
        _ptr(k_src), _ptr(v_src), pitch, _ptr(rope), rope.shape[0], ctypes.c_float(eps),
        _ptr(pos), dtype)


def matmul_nt(a, b_nt, dtype):
    """a: [m, k], b_nt: [n, k] storage arrays -> float32 [m, n], binary32 accumulation."""
    m, k = a.shape
    n = b_nt.shape[0]
    c = np.zeros((m, n), dtype=np.float32)
    load().ellm_oracle_matmul_nt(_ptr(a), _ptr(b_nt), _ptr(c), m, n, k, dtype)
    return c


def matmul3(hidden, wq, wk, wv, q_state, k_state, v_state, rope, kv_strides, capacity, position_index,
            interval, dtype, batch_size=None, positions=None, eps=1e-6, rope_position_stride=128,
            rope_head_stride=0, head=128):
    """hidden: [interval_capacity, batch_pitch, k]; weights: [heads * head, k]; q_state:
    [interval_capacity, batch_pitch, q_heads, head]; k_state / v_state: storage arrays addressed
    through kv_strides (elements), all written in place.  Returns the oracle's status."""
    pitch, k = hidden.shape[1], hidden.shape[2]
    if batch_size is None:
        batch_size = pitch
    pos = np.ascontiguousarray(positions, dtype=np.uint32) if positions is not None else None
    strides = (ctypes.c_size_t * 4)(*[int(x) for x in kv_strides])
    return load().ellm_oracle_matmul3(
        _ptr(hidden), _ptr(wq), _ptr(wk), _ptr(wv), _ptr(q_state), _ptr(k_state), _ptr(v_state),
        _ptr(rope), rope_position_stride, rope_head_stride, rope.size, k, pitch, batch_size,
        wq.shape[0] // head, wk.shape[0] // head, head, ctypes.byref(strides), capacity,
        position_index, interval, _ptr(pos), ctypes.c_float(eps), dtype)


def matmul_add(a, b_nt, residual, dtype, interval=None, batch_size=None):
    """a: [interval_capacity, batch_pitch, k]; b_nt: [n, k]; residual: [.., .., n] -> output."""
    pitch, k = a.shape[1], a.shape[2]
    n = b_nt.shape[0]
    out = np.zeros_like(residual)
    load().ellm_oracle_matmul_add(_ptr(a), _ptr(b_nt), _ptr(residual), _ptr(out), n, k, pitch,
                                  batch_size if batch_size is not None else pitch,
                                  interval if interval is not None else a.shape[0], dtype)
    return out


def assign(length, num, idx):
    lib = load()
    b, e = ctypes.c_size_t(), ctypes.c_size_t()
    ok = lib.ellm_oracle_assign(length, num, idx, ctypes.byref(b), ctypes.byref(e))
    return (b.value, e.value) if ok else None


def flash_attention_row(q, K, V, scale, position, dtype, stride=None, o_init=None):
    """One query row against rows 0..=position of K/V (storage arrays). Returns (o, lse)."""
    lib = load()
    length = q.shape[-1]
    stride = stride if stride is not None else length
    o = np.zeros(length, dtype=storage_np_dtype(dtype)) if o_init is None else o_init.copy()
    lse = np.zeros(1, dtype=np.float32)
    lib.ellm_oracle_flash_attention(_ptr(q), _ptr(K), _ptr(V), _ptr(o), _ptr(lse),
                                    ctypes.c_float(scale), length, stride, position, dtype)
    return o, float(lse[0])


class Operator:
    """The oracle's Attention operator over numpy storage arrays.

    q/out: [interval, batch_capacity, heads, D]; k/v: [sequence, kv_head, capacity, D]
    (or any layout described by kv_strides, in elements).
    """

    def __init__(self, q, k, v, out, lse, batch_capacity, heads, kv_heads, head_size, kv_strides,
                 scale, dtype):
        self.keep = (q, k, v, out, lse)
        d = OracleAttn()
        d.q, d.k, d.v, d.out = q.ctypes.data, k.ctypes.data, v.ctypes.data, out.ctypes.data
        d.lse = lse.ctypes.data if lse is not None else None
        d.batch_capacity, d.attention_head_num, d.kv_head_num, d.head_size = (
            batch_capacity, heads, kv_heads, head_size)
        for i in range(4):
            d.kv_strides[i] = int(kv_strides[i])
        d.inverse_sqrt_head = scale
        d.dtype = dtype
        self.desc = d

    def run(self, position_index, position_interval, batch_size, cpu_num=1, thread_id=0,
            positions=None):
        rc = load().ellm_oracle_attention_run(ctypes.byref(self.desc), position_index,
                                              position_interval, batch_size, _ptr(positions),
                                              cpu_num, thread_id)
        if rc:
            raise RuntimeError("oracle rejected the arguments")

    def run_threads(self, position_index, position_interval, batch_size, n_threads,
                    positions=None, pin=False, repeats=1):
        t = load().ellm_oracle_attention_run_threads(ctypes.byref(self.desc), position_index,
                                                     position_interval, batch_size,
                                                     _ptr(positions), n_threads, int(pin), repeats)
        if t < 0:
            raise RuntimeError("oracle rejected the arguments")
        return t

    def run_rows(self, position_index, rows, n_threads, positions=None, pin=False):
        """rows: uint32 [n, 3] of (token_in_chunk, sequence, head); positions: optional uint32
        per-sequence positions (single-token steps). Returns (out_rows, lse, secs)."""
        rows = np.ascontiguousarray(rows, dtype=np.uint32)
        n = rows.shape[0]
        out = np.zeros((n, self.desc.head_size), dtype=storage_np_dtype(self.desc.dtype))
        lse = np.zeros(n, dtype=np.float32)
        if positions is not None:
            positions = np.ascontiguousarray(positions, dtype=np.uint32)
        t = load().ellm_oracle_attention_rows_threads_ex(ctypes.byref(self.desc), position_index,
                                                         _ptr(positions), _ptr(rows), n, _ptr(out),
                                                         _ptr(lse), n_threads, int(pin))
        if t < 0:
            raise RuntimeError("oracle rejected the arguments")
        return out, lse, t


def attention(q, k, v, scale, dtype, position_index=0, positions=None, n_threads=8, batch=None):
    """Convenience: run the whole operator on numpy storage arrays.

    q: [S, Bcap, Hq, D]; k, v: [B, Hkv, cap, D] contiguous.  Returns (out, lse[S, Bcap, Hq]).
    """
    S, bcap, hq, D = q.shape
    hkv, cap = k.shape[1], k.shape[2]
    out = np.zeros_like(q)
    lse = np.zeros((S, bcap, hq), dtype=np.float32)
    op = Operator(q, k, v, out, lse, bcap, hq, hkv, D, [hkv * cap * D, cap * D, D, 1], scale, dtype)
    op.run_threads(position_index, S, batch if batch is not None else bcap, n_threads,
                   positions=positions)
    return out, lse
