"""ctypes declarations for the C ABI in ``include/ellm_attn.h``."""
import ctypes
import os

DTYPE_F16 = 0
DTYPE_BF16 = 1
DTYPE_F32 = 2   # attention only

_HERE = os.path.dirname(os.path.abspath(__file__))


def lib_path():
    return os.path.join(_HERE, "lib", "libellm_attn.so")


class LibraryMissing(RuntimeError):
    """libellm_attn.so has not been built (run ``__graft_entry__.build()``)."""


class EllmError(RuntimeError):
    def __init__(self, status, message):
        super().__init__(f"ellm status {status}: {message}")
        self.status = status
        self.message = message


class AttnDesc(ctypes.Structure):
    _fields_ = [
        ("q", ctypes.c_void_p),
        ("k", ctypes.c_void_p),
        ("v", ctypes.c_void_p),
        ("out", ctypes.c_void_p),
        ("lse", ctypes.c_void_p),
        ("batch_size", ctypes.c_size_t),
        ("attention_head_num", ctypes.c_size_t),
        ("kv_head_num", ctypes.c_size_t),
        ("head_size", ctypes.c_size_t),
        ("kv_strides", ctypes.c_size_t * 4),
        ("inverse_sqrt_head", ctypes.c_float),
        ("dtype", ctypes.c_int),
        ("sequence_capacity", ctypes.c_size_t),
        ("max_position_interval", ctypes.c_size_t),
    ]


class KvDesc(ctypes.Structure):
    _fields_ = [
        ("layers", ctypes.c_size_t),
        ("sequences", ctypes.c_size_t),
        ("kv_head_num", ctypes.c_size_t),
        ("head_size", ctypes.c_size_t),
        ("capacity", ctypes.c_size_t),
        ("dtype", ctypes.c_int),
    ]


class KvRaggedDesc(ctypes.Structure):
    _fields_ = [
        ("layers", ctypes.c_size_t),
        ("sequences", ctypes.c_size_t),
        ("kv_head_num", ctypes.c_size_t),
        ("head_size", ctypes.c_size_t),
        ("capacities", ctypes.POINTER(ctypes.c_size_t)),
        ("dtype", ctypes.c_int),
    ]


class KvSeqTable(ctypes.Structure):
    _fields_ = [
        ("seq_offsets", ctypes.c_void_p),
        ("seq_capacity", ctypes.c_void_p),
        ("seq_capacity_host", ctypes.POINTER(ctypes.c_size_t)),
        ("sequences", ctypes.c_size_t),
    ]


class MatMul3Desc(ctypes.Structure):
    _fields_ = [
        ("hidden", ctypes.c_void_p),
        ("q_weight", ctypes.c_void_p),
        ("k_weight", ctypes.c_void_p),
        ("v_weight", ctypes.c_void_p),
        ("q_state", ctypes.c_void_p),
        ("k_state", ctypes.c_void_p),
        ("v_state", ctypes.c_void_p),
        ("rope", ctypes.c_void_p),
        ("rope_position_stride", ctypes.c_size_t),
        ("rope_head_stride", ctypes.c_size_t),
        ("rope_elems", ctypes.c_size_t),
        ("hidden_size", ctypes.c_size_t),
        ("batch_size", ctypes.c_size_t),
        ("attention_head_num", ctypes.c_size_t),
        ("kv_head_num", ctypes.c_size_t),
        ("head_size", ctypes.c_size_t),
        ("kv_strides", ctypes.c_size_t * 4),
        ("sequence_capacity", ctypes.c_size_t),
        ("max_position_interval", ctypes.c_size_t),
        ("eps", ctypes.c_float),
        ("dtype", ctypes.c_int),
    ]


class MatMulAddDesc(ctypes.Structure):
    _fields_ = [
        ("a", ctypes.c_void_p),
        ("b_nt", ctypes.c_void_p),
        ("residual", ctypes.c_void_p),
        ("output", ctypes.c_void_p),
        ("batch_size", ctypes.c_size_t),
        ("n", ctypes.c_size_t),
        ("k", ctypes.c_size_t),
        ("max_position_interval", ctypes.c_size_t),
        ("dtype", ctypes.c_int),
    ]


_sz = ctypes.c_size_t
_vp = ctypes.c_void_p
_pvp = ctypes.POINTER(ctypes.c_void_p)

# name -> (restype, argtypes); every entry point include/ellm_attn.h declares.
ABI_SYMBOLS = {
    "ellm_last_error_string": (ctypes.c_char_p, []),
    "ellm_attn_version": (ctypes.c_int, []),
    "ellm_device_count": (ctypes.c_int, []),
    "ellm_attn_create": (ctypes.c_int, [ctypes.POINTER(AttnDesc), _pvp]),
    "ellm_attn_destroy": (ctypes.c_int, [_vp]),
    "ellm_attn_reset": (ctypes.c_int, [_vp, _vp]),
    "ellm_matmul3_reset": (ctypes.c_int, [_vp, _vp]),
    "ellm_matmul_add_reset": (ctypes.c_int, [_vp, _vp]),
    "ellm_attn_run": (ctypes.c_int, [_vp, _sz, _sz, _sz, _vp]),
    "ellm_attn_run_ragged": (ctypes.c_int, [_vp, _vp, _sz, _sz, _vp]),
    "ellm_attn_ragged_path": (ctypes.c_int, [_vp, _sz, _sz]),
    "ellm_attn_run_noalloc": (ctypes.c_int, [ctypes.POINTER(AttnDesc), _vp, _sz, _sz, _vp]),
    "ellm_kv_create": (ctypes.c_int, [ctypes.POINTER(KvDesc), _pvp]),
    "ellm_kv_create_ragged": (ctypes.c_int, [ctypes.POINTER(KvRaggedDesc), _pvp]),
    "ellm_kv_layer_ragged": (ctypes.c_int, [_vp, _sz, _sz, _pvp, _pvp, ctypes.POINTER(_sz * 4),
                                            ctypes.POINTER(KvSeqTable)]),
    "ellm_attn_create_ragged": (ctypes.c_int, [ctypes.POINTER(AttnDesc), ctypes.POINTER(KvSeqTable), _pvp]),
    "ellm_matmul3_create_ragged": (ctypes.c_int, [ctypes.POINTER(MatMul3Desc), ctypes.POINTER(KvSeqTable),
                                                  _pvp]),
    "ellm_kv_destroy": (ctypes.c_int, [_vp]),
    "ellm_kv_layer": (ctypes.c_int, [_vp, _sz, _pvp, _pvp, ctypes.POINTER(_sz * 4)]),
    "ellm_kv_append": (ctypes.c_int, [_vp, _sz, _sz, _sz, _sz, _vp, _vp, _sz, _vp]),
    "ellm_kv_append_norm_rope": (ctypes.c_int, [_vp, _sz, _sz, _sz, _sz, _vp, _vp, _sz, _vp, _sz,
                                                ctypes.c_float, _vp, _sz, _vp]),
    "ellm_kv_append_attn_run": (ctypes.c_int, [_vp, _sz, _vp, _sz, _sz, _vp, _vp, _vp, _sz, ctypes.c_float, _vp]),
    "ellm_kv_append_attn_run_ragged": (ctypes.c_int, [_vp, _sz, _vp, _vp, _sz, _sz, _vp, _vp, _vp, _sz,
                                                      ctypes.c_float, _vp]),
    "ellm_schedule_calls": (ctypes.c_int, [_sz, _sz, _sz, _sz, _vp, _sz, ctypes.POINTER(_sz)]),
    "ellm_graph_begin": (ctypes.c_int, [_vp]),
    "ellm_graph_end": (ctypes.c_int, [_vp, _pvp]),
    "ellm_graph_launch": (ctypes.c_int, [_vp, _vp]),
    "ellm_graph_destroy": (ctypes.c_int, [_vp]),
    "ellm_side_stream_create": (ctypes.c_int, [_pvp]),
    "ellm_side_stream_get": (ctypes.c_void_p, [_vp]),
    "ellm_side_stream_fork": (ctypes.c_int, [_vp, _vp]),
    "ellm_side_stream_join": (ctypes.c_int, [_vp, _vp]),
    "ellm_side_stream_destroy": (ctypes.c_int, [_vp]),
    "ellm_positions_advance": (ctypes.c_int, [_vp, _sz, ctypes.c_uint32, _vp]),
    "ellm_matmul3_create": (ctypes.c_int, [ctypes.POINTER(MatMul3Desc), _pvp]),
    "ellm_matmul3_run": (ctypes.c_int, [_vp, _sz, _sz, _sz, _vp]),
    "ellm_matmul3_run_ragged": (ctypes.c_int, [_vp, _vp, _sz, _sz, _vp]),
    "ellm_matmul3_destroy": (ctypes.c_int, [_vp]),
    "ellm_matmul3_attn_run": (ctypes.c_int, [_vp, _vp, _sz, _sz, _vp]),
    "ellm_matmul3_attn_run_ragged": (ctypes.c_int, [_vp, _vp, _vp, _sz, _sz, _vp]),
    "ellm_matmul3_attn_path": (ctypes.c_int, [_vp, _vp, _sz]),
    "ellm_matmul_add_create": (ctypes.c_int, [ctypes.POINTER(MatMulAddDesc), _pvp]),
    "ellm_matmul_add_run": (ctypes.c_int, [_vp, _sz, _sz, _sz, _vp]),
    "ellm_matmul_add_destroy": (ctypes.c_int, [_vp]),
    "ellm_projection_path": (ctypes.c_int, [_sz, _sz, _sz]),
}

_lib = None


def load_library():
    """Load libellm_attn.so once; raises LibraryMissing when it is not built."""
    global _lib
    if _lib is not None:
        return _lib
    path = lib_path()
    if not os.path.exists(path):
        raise LibraryMissing(f"{path} not found; build it with __graft_entry__.build()")
    # PyTorch carries a HIP runtime of its own under the same soname.  A process that
    # loaded the system's runtime first and PyTorch's second holds two runtimes, and the
    # one that reaches the device second finds none ("no ROCm-capable device is
    # detected").  Importing torch first makes the library bind to the runtime torch
    # uses, so the tensors whose addresses it is given and its own calls share one.
    try:
        import torch  # noqa: F401
    except ImportError:
        pass  # a host without PyTorch uses the system's runtime alone
    lib = ctypes.CDLL(path)
    for name, (res, args) in ABI_SYMBOLS.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def check(status):
    if status != 0:
        msg = load_library().ellm_last_error_string()
        raise EllmError(status, msg.decode() if msg else "")
