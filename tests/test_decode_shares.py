"""The share arithmetic of the single-token kernel for sequences of different lengths
(ellm_amd/csrc/decode_shares.hpp, 32-bit with one double-precision estimate) against 64-bit integer
arithmetic, on the host: share g begins at floor(g U / W); holder(unit) is the share that contains it;
runs of equal length end on share ends when W is a multiple of their number."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "ellm_amd", "csrc")

PROBE = r"""
#include "decode_shares.hpp"
#include <cstdio>
using namespace ellm;
int main() {
  unsigned long long checked = 0, bad = 0;
  const uint32_t Ws[] = {1, 2, 7, 8, 96, 480, 500, 512, 1000, 65535};
  const uint32_t Us[] = {1, 5, 511, 512, 513, 12288, 141104, 1000003, (1u << 31) - 70000u};
  for (uint32_t W : Ws) for (uint32_t U : Us) {
    if (W > U) continue;
    const Shares s(W, U);
    for (uint32_t g = 0; g <= W; g += (W > 2000 ? 37 : 1)) {
      bad += s.begin(g) != (uint32_t)(((unsigned long long)g * U) / W);
      ++checked;
    }
    const uint32_t step = U > 200000 ? U / 100003 + 1 : 1;
    for (unsigned long long u = 0; u < U; u += step) {
      const uint32_t g = s.holder((uint32_t)u);
      bad += !(g < W && s.begin(g) <= u && s.begin(g + 1) > u);
      ++checked;
    }
    for (uint32_t g = 0; g < W; g += (W > 2000 ? 997 : 1)) {       // first and last unit of a share
      if (s.begin(g + 1) == s.begin(g)) continue;
      bad += s.holder(s.begin(g)) != g;
      bad += s.holder(s.begin(g + 1) - 1) != g;
      checked += 2;
    }
  }
  // 96 runs of 128 units on 480 workgroups: every run is five whole shares
  const Shares t(480, 96 * 128);
  for (uint32_t p = 0; p <= 96; ++p) bad += t.begin(5 * p) != 128 * p;
  printf("%llu %llu\n", checked, bad);
  return 0;
}
"""


def test_shares_match_64_bit_arithmetic(tmp_path):
    gxx = shutil.which("g++")
    if not gxx:
        pytest.skip("no g++")
    src = tmp_path / "probe.cpp"
    src.write_text(PROBE)
    exe = tmp_path / "probe"
    subprocess.run([gxx, "-O2", "-std=c++17", "-I", CSRC, str(src), "-o", str(exe)], check=True, timeout=300)
    checked, bad = (int(x) for x in subprocess.run([str(exe)], check=True, capture_output=True, text=True,
                                                   timeout=300).stdout.split())
    assert checked > 1_000_000 and bad == 0
