"""Argument checking of the projection entry points: descriptions are rejected before
anything touches a device; the range checks of run need a handle (and so a device) but
launch nothing and never dereference the pointers."""
import ctypes

import pytest

import ellm_amd
from ellm_amd import _lib

OK, INVALID, UNSUPPORTED, OUT_OF_RANGE, NO_DEVICE = 0, 1, 2, 3, 5


def _m3(**over):
    d = _lib.MatMul3Desc()
    for name in ("hidden", "q_weight", "k_weight", "v_weight", "q_state", "k_state", "v_state", "rope"):
        setattr(d, name, 0x1000)
    d.rope_position_stride, d.rope_head_stride, d.rope_elems = 128, 0, 64 * 128
    d.hidden_size, d.batch_size, d.attention_head_num, d.kv_head_num, d.head_size = 256, 2, 8, 2, 128
    for i, s in enumerate((2 * 64 * 128, 64 * 128, 128, 1)):
        d.kv_strides[i] = s
    d.sequence_capacity, d.max_position_interval, d.eps, d.dtype = 64, 16, 1e-6, _lib.DTYPE_F16
    for k, v in over.items():
        if k == "kv_strides":
            for i, s in enumerate(v):
                d.kv_strides[i] = s
        else:
            setattr(d, k, v)
    return d


@pytest.mark.parametrize("over,status", [
    (dict(hidden=None), INVALID),
    (dict(rope=0x1004), INVALID),
    (dict(dtype=3), INVALID),
    (dict(head_size=64), UNSUPPORTED),
    (dict(hidden_size=96), UNSUPPORTED),                 # not a multiple of 64
    (dict(kv_head_num=0), INVALID),
    (dict(kv_strides=(2 * 64 * 128, 64 * 128, 128, 2)), INVALID),
    (dict(rope_position_stride=130), INVALID),
    (dict(rope_elems=64), INVALID),
    (dict(eps=float("nan")), INVALID),
])
def test_matmul3_create(over, status):
    lib = ellm_amd.load_library()
    h = ctypes.c_void_p()
    assert lib.ellm_matmul3_create(ctypes.byref(_m3(**over)), ctypes.byref(h)) == status
    assert not h.value


def test_matmul3_create_ragged_rejects_a_zero_capacity():
    """The kernels clamp a position to capacity - 1; a capacity of 0 would wrap and switch the clamp
    off.  Refused before anything touches a device, as ellm_attn_create_ragged does."""
    lib = ellm_amd.load_library()
    caps = (ctypes.c_size_t * 2)(64, 0)
    table = _lib.KvSeqTable()
    table.seq_offsets = 0x1000
    table.seq_capacity = 0x2000
    table.seq_capacity_host = ctypes.cast(caps, ctypes.POINTER(ctypes.c_size_t))
    table.sequences = 2
    h = ctypes.c_void_p()
    assert lib.ellm_matmul3_create_ragged(ctypes.byref(_m3()), ctypes.byref(table), ctypes.byref(h)) == INVALID
    assert b"capacity 0" in lib.ellm_last_error_string() and not h.value


def test_create_without_a_device_says_so():
    lib = ellm_amd.load_library()
    if lib.ellm_device_count() > 0:
        pytest.skip("a device is present")
    h = ctypes.c_void_p()
    assert lib.ellm_matmul3_create(ctypes.byref(_m3()), ctypes.byref(h)) == NO_DEVICE and not h.value
    assert lib.ellm_matmul_add_create(ctypes.byref(_ma()), ctypes.byref(h)) == NO_DEVICE and not h.value


@pytest.mark.gpu
def test_matmul3_run_range_checks():
    lib = ellm_amd.load_library()
    h = ctypes.c_void_p()
    assert lib.ellm_matmul3_create(ctypes.byref(_m3()), ctypes.byref(h)) == OK
    assert lib.ellm_matmul3_run(h, 0, 17, 2, None) == OUT_OF_RANGE       # interval beyond the maximum
    assert lib.ellm_matmul3_run(h, 0, 1, 3, None) == OUT_OF_RANGE        # batch beyond the capacity
    assert lib.ellm_matmul3_run(h, 60, 5, 2, None) == OUT_OF_RANGE       # position 64 of 64
    assert b"outside the cache" in lib.ellm_last_error_string()
    assert lib.ellm_matmul3_run(h, 0, 0, 2, None) == OK                  # nothing to do
    assert lib.ellm_matmul3_run_ragged(h, None, 10, 2, None) == INVALID
    assert lib.ellm_matmul3_run_ragged(h, 0x1000, 64, 2, None) == OUT_OF_RANGE
    assert lib.ellm_matmul3_destroy(h) == OK
    # a table shorter than the cache bounds the positions too
    assert lib.ellm_matmul3_create(ctypes.byref(_m3(rope_elems=8 * 128)), ctypes.byref(h)) == OK
    assert lib.ellm_matmul3_run(h, 7, 2, 2, None) == OUT_OF_RANGE
    assert b"rotary table" in lib.ellm_last_error_string()
    assert lib.ellm_matmul3_destroy(h) == OK


def _ma(**over):
    d = _lib.MatMulAddDesc()
    d.a = d.b_nt = d.residual = d.output = 0x1000
    d.batch_size, d.n, d.k, d.max_position_interval, d.dtype = 4, 256, 128, 8, _lib.DTYPE_BF16
    for k, v in over.items():
        setattr(d, k, v)
    return d


@pytest.mark.parametrize("over,status", [
    (dict(output=None), INVALID),
    (dict(a=0x1008), INVALID),
    (dict(n=200), UNSUPPORTED),
    (dict(k=100), UNSUPPORTED),
    (dict(batch_size=0), INVALID),
    (dict(dtype=-1), INVALID),
])
def test_matmul_add_create(over, status):
    lib = ellm_amd.load_library()
    h = ctypes.c_void_p()
    assert lib.ellm_matmul_add_create(ctypes.byref(_ma(**over)), ctypes.byref(h)) == status
    assert not h.value


@pytest.mark.gpu
def test_matmul_add_run_range_checks():
    lib = ellm_amd.load_library()
    h = ctypes.c_void_p()
    assert lib.ellm_matmul_add_create(ctypes.byref(_ma()), ctypes.byref(h)) == OK
    assert lib.ellm_matmul_add_run(h, 0, 9, 4, None) == OUT_OF_RANGE
    assert lib.ellm_matmul_add_run(h, 0, 1, 5, None) == OUT_OF_RANGE
    assert lib.ellm_matmul_add_run(h, 0, 0, 4, None) == OK
    assert lib.ellm_matmul_add_destroy(h) == OK


def test_projection_path_rule():
    """ellm_projection_path without a device (256 compute units assumed): the few-rows kernel up
    to 64 rows when K suits it, then the smallest one-head tile whose workgroups fit the part in
    one round, then the 256 x 256 tiles; sizes no handle accepts give -1."""
    lib = ellm_amd.load_library()
    path = lib.ellm_projection_path
    few, t128, t256, big = 0, 1, 2, 3
    assert path(1, 40, 2048) == few and path(64, 40, 2048) == few
    assert path(65, 40, 2048) == t128                 # one 128-token tile per head
    assert path(16, 40, 64) == t128                   # K too short for the streaming kernel's waves
    assert path(6 * 128, 40, 2048) == t128 and path(6 * 128 + 1, 40, 2048) == t256
    assert path(6 * 256, 40, 2048) == t256 and path(6 * 256 + 1, 40, 2048) == big
    assert path(16 * 128, 16, 4096) == t128 and path(16 * 256, 16, 4096) == t256
    assert path(16 * 256 + 1, 16, 4096) == big and path(32768, 40, 2048) == big
    assert path(0, 40, 2048) == -1 and path(16, 0, 2048) == -1 and path(16, 40, 0) == -1
    assert path(1 << 40, 40, 2048) == -1 and path(16, 40, 1 << 20) == -1
