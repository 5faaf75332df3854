"""The C ABI without a GPU: the library loads, exports every symbol the header
declares, and rejects bad descriptions with a status instead of aborting
(the reference has no error path at all: src/compiler/operator.rs:243 panics,
Cargo.toml:49 makes a panic an abort)."""
import ctypes
import os
import re

import pytest

import ellm_amd
from ellm_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

OK, INVALID, UNSUPPORTED, OUT_OF_RANGE, HIP, NO_DEVICE = range(6)


def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "ellm_attn.h")).read()
    header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
    declared = set(re.findall(r"\b(ellm_[a-z_0-9]+)\s*\(", header))
    assert declared == set(_lib.ABI_SYMBOLS), declared ^ set(_lib.ABI_SYMBOLS)
    lib = ctypes.CDLL(ellm_amd.lib_path())
    for name in declared:
        assert getattr(lib, name) is not None


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "lib_path", lambda: str(tmp_path / "nope.so"))
    with pytest.raises(ellm_amd.LibraryMissing):
        _lib.load_library()


def test_loading_before_torch_leaves_one_hip_runtime_in_the_process():
    """A process that loads the library before it imports torch must not end up with the
    system's HIP runtime beside PyTorch's own copy: the second of two runtimes to reach
    the device finds none."""
    import subprocess
    import sys
    code = (
        "import ellm_amd\n"
        "ellm_amd.load_library()\n"
        "import torch\n"
        "paths = {l.split()[-1] for l in open('/proc/self/maps') if 'libamdhip64' in l}\n"
        "print(len(paths), sorted(paths))\n"
    )
    r = subprocess.run([sys.executable, "-c", code], cwd=ROOT, capture_output=True, text=True,
                       timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    assert r.stdout.split()[0] == "1", r.stdout


def test_version_and_device_count():
    lib = ellm_amd.load_library()
    assert lib.ellm_attn_version() >= 100
    assert lib.ellm_device_count() >= 0


def _desc(**over):
    d = _lib.AttnDesc()
    d.q = d.k = d.v = d.out = 0x1000
    d.lse = None
    d.batch_size, d.attention_head_num, d.kv_head_num, d.head_size = 2, 8, 2, 128
    for i, s in enumerate((2 * 64 * 128, 64 * 128, 128, 1)):
        d.kv_strides[i] = s
    d.inverse_sqrt_head = 0.088
    d.dtype = _lib.DTYPE_F16
    d.sequence_capacity, d.max_position_interval = 64, 16
    for k, v in over.items():
        if k == "kv_strides":
            for i, s in enumerate(v):
                d.kv_strides[i] = s
        else:
            setattr(d, k, v)
    return d


@pytest.mark.parametrize("over,status", [
    (dict(q=None), INVALID),
    (dict(out=None), INVALID),
    (dict(k=0x1008), INVALID),                       # not 16-byte aligned
    (dict(dtype=7), INVALID),
    (dict(head_size=0), UNSUPPORTED),
    (dict(head_size=257), UNSUPPORTED),              # the plain kernel's lanes hold four elements each
    (dict(head_size=64, kv_strides=(2 * 64 * 64, 64 * 64, 32, 1)), INVALID),   # rows closer than a head
    (dict(dtype=3), INVALID),
    (dict(attention_head_num=7), INVALID),           # not a multiple of kv_head_num
    (dict(kv_head_num=0), INVALID),
    (dict(kv_strides=(2 * 64 * 128, 64 * 128, 128, 2)), INVALID),
    (dict(kv_strides=(2 * 64 * 128, 64 * 128, 100, 1)), INVALID),
    (dict(sequence_capacity=0), INVALID),
    (dict(max_position_interval=65), INVALID),
    (dict(inverse_sqrt_head=float("nan")), INVALID),
])
def test_create_rejects_bad_descriptions(over, status):
    lib = ellm_amd.load_library()
    h = ctypes.c_void_p()
    rc = lib.ellm_attn_create(ctypes.byref(_desc(**over)), ctypes.byref(h))
    assert rc == status
    assert not h.value
    assert lib.ellm_last_error_string()


def test_null_arguments():
    lib = ellm_amd.load_library()
    h = ctypes.c_void_p()
    assert lib.ellm_attn_create(None, ctypes.byref(h)) == INVALID
    assert lib.ellm_attn_run(None, 0, 1, 1, None) == INVALID
    assert lib.ellm_attn_run_ragged(None, None, 0, 1, None) == INVALID
    assert lib.ellm_attn_destroy(None) == OK
    assert lib.ellm_kv_destroy(None) == OK
    assert lib.ellm_kv_append_attn_run(None, 0, None, 0, 1, None, None, None, 0, 1e-6, None) == INVALID
    assert lib.ellm_kv_append_attn_run_ragged(None, 0, None, None, 0, 1, None, None, None, 0, 1e-6, None) == INVALID
    assert lib.ellm_matmul3_attn_run(None, None, 0, 1, None) == INVALID
    c = ctypes.c_void_p()
    assert lib.ellm_kv_create(None, ctypes.byref(c)) == INVALID
    kd = _lib.KvDesc(1, 1, 1, 64, 16, 0)
    assert lib.ellm_kv_create(ctypes.byref(kd), ctypes.byref(c)) == UNSUPPORTED
    kd = _lib.KvDesc(0, 1, 1, 128, 16, 0)
    assert lib.ellm_kv_create(ctypes.byref(kd), ctypes.byref(c)) == INVALID
    # a size that does not fit 64 bits is refused before anything is allocated
    kd = _lib.KvDesc(1 << 40, 65535, 65535, 128, (1 << 31) - 1, 0)
    assert lib.ellm_kv_create(ctypes.byref(kd), ctypes.byref(c)) == UNSUPPORTED
    assert b"64 bits" in lib.ellm_last_error_string()


def test_valid_description_without_a_device_reports_no_device():
    lib = ellm_amd.load_library()
    if lib.ellm_device_count() > 0:
        pytest.skip("a device is present")
    h = ctypes.c_void_p()
    assert lib.ellm_attn_create(ctypes.byref(_desc()), ctypes.byref(h)) in (NO_DEVICE, HIP)
    assert not h.value


def test_host_mirror_only_thread_zero_launches():
    """Every worker thread calls run() in the reference (src/serving/start.rs:69-73);
    here all but thread 0 must return without touching the library."""
    op = ellm_amd.Attention.__new__(ellm_amd.Attention)
    op._handle = None
    op._lib = None
    op.run(0, 1, 1, cpu_num=8, thread_id=3)   # would raise if it reached the library


def test_host_mirrors_refuse_host_memory_and_wrong_types():
    """The mirrors hand raw addresses to the library: a host tensor or a tensor of another
    type must be refused on the host, before any handle exists."""
    import torch

    q = torch.zeros((1, 1, 2, 128), dtype=torch.float16)
    kv = torch.zeros((1, 1, 16, 128), dtype=torch.float16)
    with pytest.raises(TypeError, match="device"):
        ellm_amd.Attention(q, kv, kv, q.clone(), 1, 2, 1, 128, [16 * 128, 16 * 128, 128, 1], 0.1)
    x = torch.zeros((1, 1, 256), dtype=torch.float16)
    w = torch.zeros((128, 256), dtype=torch.float16)
    with pytest.raises(TypeError, match="device"):
        ellm_amd.MatMulAdd(x, w, torch.zeros((1, 1, 128), dtype=torch.float16),
                           torch.zeros((1, 1, 128), dtype=torch.float16))
    with pytest.raises(TypeError, match="device"):
        ellm_amd.MatMul3(x, w, q, w, kv, w, kv, torch.zeros((16, 128), dtype=torch.float16), 128, 1,
                         1, 1, [16 * 128, 16 * 128, 128, 1], 16)


def test_diagnostic_library_exports_its_declared_symbol():
    """libellm_diag.so (the MFMA-stream measurement aid bench.py uses) loads without a GPU and
    exports what include/ellm_diag.h declares; it rejects bad arguments before any launch."""
    header = open(os.path.join(ROOT, "include", "ellm_diag.h")).read()
    header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
    declared = set(re.findall(r"\b(ellm_[a-z_0-9]+)\s*\(", header))
    assert declared == {"ellm_diag_mfma_stream"}
    lib = ctypes.CDLL(os.path.join(ROOT, "ellm_amd", "lib", "libellm_diag.so"))
    fn = lib.ellm_diag_mfma_stream
    fn.restype = ctypes.c_int
    fn.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int,
                   ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p]
    assert fn(0, 0, None, None, 1, 1, None, None) == 1
    assert fn(7, 0, 0x1000, 0x1000, 1, 1, None, None) == 1
