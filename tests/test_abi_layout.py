"""What a foreign-language binding depends on, checked without a GPU:

* every `typedef struct` of include/ellm_attn.h has the size and field offsets that the
  ctypes mirrors (ellm_amd/_lib.py) and the Rust `#[repr(C)]` structs
  (bindings/rust/src/lib.rs, shipped as source, not compiled here) assume — measured by a C
  probe generated from the header and compiled with g++;
* the Rust `extern "C"` block declares exactly the functions the header declares, with the
  same number of parameters;
* the CPU oracle runs clean under AddressSanitizer + UndefinedBehaviorSanitizer on buffers
  of exactly the entitled size (host code only).
"""
import ctypes
import os
import re
import subprocess

import pytest

from ellm_amd import _lib
from ellm_amd import schedule as _schedule

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "ellm_attn.h")
RUST = os.path.join(ROOT, "bindings", "rust", "src", "lib.rs")


def _strip_comments(text):
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return re.sub(r"//[^\n]*", "", text)


def _header_structs():
    """{struct name: [(field name, array length or 0)]} for every typedef struct with a body."""
    text = _strip_comments(open(HEADER).read())
    out = {}
    for m in re.finditer(r"typedef\s+struct\s+(\w+)\s*\{(.*?)\}\s*(\w+)\s*;", text, flags=re.S):
        fields = []
        for decl in m.group(2).split(";"):
            decl = decl.strip()
            if not decl:
                continue
            fm = re.match(r".*?(\w+)\s*(?:\[(\d+)\])?$", decl, flags=re.S)
            fields.append((fm.group(1), int(fm.group(2) or 0)))
        out[m.group(3)] = fields
    return out


@pytest.fixture(scope="module")
def c_layout(tmp_path_factory):
    """{struct: {"sizeof": n, field: (offset, size)}} as the C compiler lays the header out."""
    structs = _header_structs()
    lines = ['#include <stddef.h>', '#include <stdio.h>', f'#include "{HEADER}"', "int main(void) {"]
    for name, fields in structs.items():
        lines.append(f'  printf("{name} sizeof %zu\\n", sizeof({name}));')
        for field, _ in fields:
            lines.append(f'  printf("{name} {field} %zu %zu\\n", offsetof({name}, {field}), '
                         f'sizeof((({name}*)0)->{field}));')
    lines += ["  return 0;", "}"]
    d = tmp_path_factory.mktemp("abi_probe")
    src, exe = d / "probe.c", d / "probe"
    src.write_text("\n".join(lines))
    # as C and as C++: the header must mean the same to both
    layouts = []
    for compiler, flags in (("gcc", ["-std=c99"]), ("g++", ["-std=c++17", "-x", "c++"])):
        subprocess.check_call([compiler, *flags, "-fsanitize=address,undefined", "-Wall", "-Werror",
                               str(src), "-o", str(exe)])
        text = subprocess.check_output([str(exe)], text=True)
        layout = {}
        for line in text.splitlines():
            parts = line.split()
            if parts[1] == "sizeof":
                layout.setdefault(parts[0], {})["sizeof"] = int(parts[2])
            else:
                layout.setdefault(parts[0], {})[parts[1]] = (int(parts[2]), int(parts[3]))
        layouts.append(layout)
    assert layouts[0] == layouts[1]
    return layouts[0]


CTYPES_MIRRORS = {
    "ellm_attn_desc": _lib.AttnDesc,
    "ellm_kv_desc": _lib.KvDesc,
    "ellm_kv_ragged_desc": _lib.KvRaggedDesc,
    "ellm_kv_seq_table": _lib.KvSeqTable,
    "ellm_matmul3_desc": _lib.MatMul3Desc,
    "ellm_matmul_add_desc": _lib.MatMulAddDesc,
    "ellm_call": _schedule._Call,
}


def test_every_header_struct_has_a_ctypes_mirror():
    assert set(_header_structs()) == set(CTYPES_MIRRORS)


@pytest.mark.parametrize("name", sorted(CTYPES_MIRRORS))
def test_ctypes_mirror_matches_the_c_layout(name, c_layout):
    mirror, want = CTYPES_MIRRORS[name], c_layout[name]
    assert ctypes.sizeof(mirror) == want["sizeof"]
    names = [f[0] for f in mirror._fields_]
    assert names == [f for f, _ in _header_structs()[name]], "field order"
    for field in names:
        desc = getattr(mirror, field)
        assert (desc.offset, desc.size) == want[field], field


# ---- the Rust source --------------------------------------------------------------------------

RUST_TYPES = {  # size, alignment on x86-64 (LP64), the only target of the library
    "usize": (8, 8), "f32": (4, 4), "c_int": (4, 4), "u32": (4, 4),
}


def _rust_type_layout(ty):
    ty = ty.strip()
    if ty.startswith("*const") or ty.startswith("*mut"):
        return 8, 8
    m = re.match(r"\[(\w+);\s*(\d+)\]", ty)
    if m:
        size, align = RUST_TYPES[m.group(1)]
        return size * int(m.group(2)), align
    return RUST_TYPES[ty]


def _rust_structs():
    text = _strip_comments(open(RUST).read())
    out = {}
    for m in re.finditer(r"#\[repr\(C\)\]\s*(?:#\[derive\([^\]]*\)\]\s*)?pub struct (\w+)\s*\{(.*?)\}", text,
                         flags=re.S):
        fields = re.findall(r"pub\s+(\w+)\s*:\s*([^,]+),", m.group(2))
        if fields:                      # opaque handles have a private zero-length member only
            out[m.group(1)] = fields
    return out


def test_rust_repr_c_structs_match_the_c_layout(c_layout):
    rust = _rust_structs()
    assert set(rust) == set(c_layout), set(rust) ^ set(c_layout)
    for name, fields in rust.items():
        want = c_layout[name]
        offset, max_align = 0, 1
        assert [f for f, _ in fields] == [f for f, _ in _header_structs()[name]], name
        for field, ty in fields:
            size, align = _rust_type_layout(ty)
            offset = (offset + align - 1) // align * align          # repr(C): C's rule
            assert (offset, size) == want[field], (name, field)
            offset += size
            max_align = max(max_align, align)
        assert (offset + max_align - 1) // max_align * max_align == want["sizeof"], name


def _split_params(params):
    return [p for p in (x.strip() for x in params.replace("\n", " ").split(",")) if p and p != "void"]


def test_rust_extern_block_declares_the_header_functions():
    header = _strip_comments(open(HEADER).read())
    declared = {m.group(1): len(_split_params(m.group(2)))
                for m in re.finditer(r"\b(ellm_[a-z_0-9]+)\s*\(([^)]*)\)\s*;", header)}
    assert set(declared) == set(_lib.ABI_SYMBOLS)
    rust = _strip_comments(open(RUST).read())
    block = re.search(r'extern "C" \{(.*?)\n\}', rust, flags=re.S).group(1)
    rust_fns = {m.group(1): len(_split_params(m.group(2)))
                for m in re.finditer(r"pub fn (ellm_[a-z_0-9]+)\s*\(([^)]*)\)", block, flags=re.S)}
    assert rust_fns == declared
    # and the ctypes table has the same arities
    assert {k: len(v[1]) for k, v in _lib.ABI_SYMBOLS.items()} == declared


def test_rust_crate_builds_the_library_with_hipcc_for_gfx950():
    build = open(os.path.join(ROOT, "bindings", "rust", "build.rs")).read()
    assert "gfx950" in build and "hipcc" in build and "rustc-link-lib=dylib=ellm_attn" in build
    for word in ("cuda", "nvcc", "hipify"):
        assert word not in build.lower()
    # every source the Makefile compiles is a rebuild trigger of the crate
    makefile = open(os.path.join(ROOT, "ellm_amd", "csrc", "Makefile")).read()
    srcs = re.search(r"^SRCS := (.*)$", makefile, flags=re.M).group(1).split()
    for s in srcs:
        assert f'"{s}"' in build, s


# ---- host-side sanitizers ------------------------------------------------------------------

def test_oracle_runs_clean_under_address_and_undefined_behaviour_sanitizers(tmp_path):
    exe = tmp_path / "oracle_asan"
    subprocess.check_call(["g++", "-std=c++17", "-O1", "-g", "-fno-omit-frame-pointer",
                           "-fsanitize=address,undefined", "-fno-sanitize-recover=all",
                           "-ffp-contract=off", "-pthread",
                           os.path.join(ROOT, "oracle", "ellm_oracle.cpp"),
                           os.path.join(ROOT, "tests", "sanitize", "oracle_driver.cpp"), "-o", str(exe)])
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0", LD_PRELOAD="")
    r = subprocess.run([str(exe)], capture_output=True, text=True, timeout=300, env=env)
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-4000:]
    assert "sanitizer run: ok" in r.stdout
