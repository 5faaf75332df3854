"""The split plan of the single-token kernel and the workspace that must hold every plan
(ellm_amd/csrc/decode_plan.hpp, host code): invariants over a sweep of shapes, and the plans of the
shapes the design quotes."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "ellm_amd", "csrc")

PROBE = r"""
#include "decode_plan.hpp"
#include <cstdio>
using namespace ellm;
int main() {
  const uint32_t lens[] = {1, 63, 64, 255, 256, 257, 1000, 2048, 4096, 8192, 40000, 65536, 131072, 1u << 20, 0x7fffffffu};
  const uint32_t heads[][2] = {{1, 1}, {8, 1}, {32, 1}, {64, 1}, {4, 4}, {32, 4}, {64, 8}, {48, 16}, {16, 16}};
  const uint32_t cus[] = {64, 256, 304};
  for (uint32_t n_cu : cus)
    for (auto& h : heads)
      for (uint32_t cap = 1; cap <= 130; cap += (cap < 34 ? 1 : 8)) {
        const DecodeWorkspace w = decode_workspace(cap, h[0], h[1], n_cu);
        for (uint32_t batch = 1; batch <= cap; batch += (batch < 34 ? 1 : 8))
          for (uint32_t len : lens) {
            const DecodePlan p = decode_plan(len, batch, h[1], n_cu);
            printf("%u %u %u %u %u %u %u %u %d\n", n_cu, h[0], h[1], cap, batch, len, p.split_len, p.n_split,
                   (int)decode_plan_fits(w, batch, h[0], h[1], h[0] / h[1], p.n_split));
          }
      }
  return 0;
}
"""


@pytest.fixture(scope="module")
def rows(tmp_path_factory):
    gxx = shutil.which("g++")
    if not gxx:
        pytest.skip("no g++")
    d = tmp_path_factory.mktemp("decode_plan")
    src = d / "probe.cpp"
    src.write_text(PROBE)
    exe = d / "probe"
    subprocess.run([gxx, "-O2", "-std=c++17", "-Wall", "-Werror", "-I", CSRC, str(src), "-o", str(exe)],
                   check=True, timeout=300)
    out = subprocess.run([str(exe)], check=True, capture_output=True, text=True, timeout=300).stdout
    return [[int(x) for x in line.split()] for line in out.splitlines()]


def test_plans_are_well_formed_and_fit_the_workspace(rows):
    assert len(rows) > 50000
    for n_cu, hq, hkv, cap, batch, length, split_len, n_split, fits in rows:
        case = (n_cu, hq, hkv, cap, batch, length, split_len, n_split)
        planes = batch * hkv
        tiny = planes * -(-length // 256) * 2 <= n_cu      # even 256-key splits would leave half of the units idle
        assert split_len % 64 == 0 and split_len >= (64 if tiny else 256), case
        if tiny and split_len < 256:
            assert n_split <= 16, case                                               # one fold
        assert n_split == -(-length // split_len) and 1 <= n_split <= 256, case     # two fold levels of 16
        assert (n_split - 1) * split_len < length, case                             # no split without keys
        assert fits == 1, case                       # the handle's workspace holds every plan it can be asked for
        if n_split > 1 and split_len > 256 and split_len * 256 > length + 64 * 256:
            # (not at one of the two floors) never more than two workgroups per compute unit
            assert planes * n_split <= 2 * n_cu, case


def test_one_workgroup_per_unit_where_the_planes_divide_the_units(rows):
    by = {(r[0], r[1], r[2], r[4], r[5]): (r[6], r[7]) for r in rows if r[3] == r[4]}
    assert by[(256, 32, 4, 16, 8192)] == (2048, 4)         # 64 planes x 4 = 256 workgroups
    assert by[(256, 32, 4, 1, 131072)] == (2048, 64)       # 4 planes x 64
    assert by[(256, 32, 4, 4, 65536)] == (4096, 16)
    assert by[(256, 32, 4, 24, 8192)] == (1664, 5)         # 96 planes: 480 workgroups on 2 x 256 beat 192 on 256
    assert by[(256, 32, 4, 20, 8192)] == (2752, 3)         # 80 planes x 3 = 240 on 256 beat 480 on 2 x 256
    assert by[(256, 32, 4, 12, 8192)] == (1664, 5)         # 48 planes x 5 = 240
    assert by[(256, 32, 4, 98, 8192)] == (8192, 1)         # more planes than units: no split
    assert by[(256, 32, 4, 1, 255)] == (64, 4)            # a tiny call: one 64-key step per workgroup
    assert by[(256, 32, 4, 4, 1000)] == (64, 16)          # 16 planes x 16 = 256 workgroups, one fold
    assert by[(256, 32, 4, 16, 1000)] == (256, 4)         # 64 planes: not tiny any more


STATIC_PROBE = r"""
#include "decode_plan.hpp"
#include <cstdio>
using namespace ellm;
int main() {
  const DecodeWorkspace room{kStaticRows, kStaticRows2, kStaticCounters};
  const uint32_t lens[] = {1, 255, 256, 257, 511, 512, 1000, 2048, 4096, 6000, 8192, 20000, 40000, 65536,
                           131072, 1u << 20, 1u << 24, 0x7fffffffu};
  const uint32_t groups[] = {1, 2, 4, 8, 16};
  const uint32_t kv[] = {1, 2, 4, 8, 16, 32};
  unsigned long n = 0, refused = 0;
  for (uint32_t g : groups)
    for (uint32_t hkv : kv)
      for (uint32_t batch = 1; batch <= 512; batch += (batch < 130 ? 1 : 16))
        for (uint32_t len : lens) {
          const uint32_t hq = g * hkv;
          const DecodePlan p = decode_plan(len, batch, hkv, 256);
          if (p.n_split == 1) continue;   // an unsplit launch touches no scratch
          const size_t rows = (size_t)batch * hq * p.n_split;
          if (rows > kStaticRows) continue;   // the documented limit
          ++n;
          const int over = decode_plan_exceeds(room, batch, hq, hkv, g, p.n_split);
          if (over) {
            ++refused;
            printf("refused %u seq x %uq/%ukv len %u: n_split %u rows %zu bound %d\n", batch, hq, hkv, len, p.n_split,
                   rows, over);
          }
        }
  printf("checked %lu refused %lu\n", n, refused);
  return 0;
}
"""


def test_static_scratch_holds_every_plan_within_its_documented_limit(tmp_path):
    """ellm_attn_run_noalloc documents one limit: sequences x query heads x splits <= 8192 partial
    rows, GQA groups of up to 16 heads.  Every plan of a 256-unit part inside that limit must fit the
    static sizes (cluster partials and counters included), or the entry point refuses shapes its
    header says it takes."""
    gxx = shutil.which("g++")
    if not gxx:
        pytest.skip("no g++")
    src = tmp_path / "probe.cpp"
    src.write_text(STATIC_PROBE)
    exe = tmp_path / "probe"
    subprocess.run([gxx, "-O2", "-std=c++17", "-Wall", "-Werror", "-I", CSRC, str(src), "-o", str(exe)],
                   check=True, timeout=300)
    out = subprocess.run([str(exe)], check=True, capture_output=True, text=True, timeout=300).stdout
    last = out.strip().splitlines()[-1].split()
    assert int(last[1]) > 3000, out[-500:]
    assert int(last[3]) == 0, out[:2000]
