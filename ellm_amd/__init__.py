"""MI355X (gfx950) attention path for eLLM: ctypes binding of ``libellm_attn.so``.

The compute lives in hand-written HIP kernels behind the C ABI declared in
``include/ellm_attn.h``; this package only loads that library and mirrors the
reference operator's interface (``Attention.new`` / ``run``) for tests and the
benchmark.  There is no CPU fallback: importing works without the library, but
any call raises :class:`LibraryMissing` until it has been built.
"""
from ._lib import (  # noqa: F401
    ABI_SYMBOLS,
    DTYPE_BF16,
    DTYPE_F16,
    DTYPE_F32,
    EllmError,
    LibraryMissing,
    lib_path,
    load_library,
)
from .attention import Attention, KVCache  # noqa: F401
from .projection import MatMul3, MatMulAdd  # noqa: F401
from .schedule import SideStream, StepGraph, positions_advance, schedule_calls  # noqa: F401
