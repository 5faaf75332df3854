"""Properties of the generated code that the sources rely on but cannot state themselves,
checked on the compiler's assembly listing (no GPU needed)."""
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "ellm_amd", "csrc")
HIPCC = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fno-strict-aliasing", "-Xclang", "-target-feature",
         "-Xclang", "-packed-fp32-ops", "-Wno-int-to-pointer-cast", "--cuda-device-only", "-S"]


def _listing(name, tmp_path):
    if not os.path.exists(HIPCC):
        pytest.skip("no hipcc")
    out = tmp_path / (name + ".s")
    subprocess.run([HIPCC, *FLAGS, "-o", str(out), os.path.join(CSRC, name)], check=True,
                   capture_output=True, timeout=600)
    return out.read_text()


def test_one_head_tile_kernels_leave_m0_to_the_inline_asm(tmp_path):
    """project_mid.hip sets M0 (the LDS address of a direct-to-LDS load) inside inline asm that
    cannot declare the write; that is sound only while the compiler keeps nothing of its own in
    M0, i.e. never indexes registers through it in these kernels."""
    text = _listing("project_mid.hip", tmp_path)
    code = [l.split(";")[0] for l in text.splitlines()]
    uses = [l for l in code if re.search(r"\bm0\b", l)]
    assert uses and all(re.fullmatch(r"\s*s_mov_b32 m0, s\d+\s*", l) for l in uses), \
        [l for l in uses if not re.fullmatch(r"\s*s_mov_b32 m0, s\d+\s*", l)][:5]
    assert not any("movrel" in l or "s_set_gpr_idx" in l for l in code)


@pytest.mark.parametrize("name", ["project.hip", "project_mid.hip", "project_small.hip", "prefill.hip", "decode.hip",
                                  "decode_balanced.hip", "kv_cache.hip"])
def test_hot_kernels_do_not_spill(name, tmp_path):
    text = _listing(name, tmp_path)
    sizes = [int(x) for x in re.findall(r"\.private_segment_fixed_size:\s*(\d+)", text)]
    assert sizes and all(v == 0 for v in sizes), sizes


def _loops(lines):
    """(first, last) line ranges of backward branches: label ... s_cbranch to that label."""
    labels = {}
    for n, l in enumerate(lines):
        m = re.match(r"^(\.LBB\d+_\d+):", l)
        if m:
            labels[m.group(1)] = n
    out = []
    for n, l in enumerate(lines):
        m = re.match(r"\s+s_cbranch_\w+\s+(\.LBB\d+_\d+)", l)
        if m and m.group(1) in labels and labels[m.group(1)] < n:
            out.append((labels[m.group(1)], n))
    return out


@pytest.mark.parametrize("name,in_loop", [("project.hip", 0)])
def test_projection_kernels_keep_scratch_out_of_their_matrix_loops(name, in_loop, tmp_path):
    """The 256 x 256 tile kernel runs at 512 registers a lane: whatever the register allocator
    does with the epilogue's values, the K loop never touches scratch (the kernel has none
    today: test_hot_kernels_do_not_spill)."""
    text = _listing(name, tmp_path)
    lines = [l.split(";")[0] for l in text.splitlines()]
    for first, last in _loops(lines):
        body = lines[first:last + 1]
        if any("v_mfma" in l for l in body):
            assert sum("scratch_" in l for l in body) <= in_loop, (name, first, last)
