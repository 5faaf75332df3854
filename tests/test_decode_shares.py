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


WALK = r"""
#include "decode_shares.hpp"
#include <cstdio>
#include <cstdlib>
#include <set>
#include <vector>
using namespace ellm;
// Walks a launch of decode_balanced.hip on the host: the workgroups that take part, the pieces each
// takes (as the kernel's loop does), the partial slot of every piece and the cluster slots of every
// plane.  Counts what the kernel relies on: every unit taken exactly once, slots distinct, at most
// 256 pieces a plane, everything inside the sizes decode_balanced_takes checks.
int main() {
  unsigned long long launches = 0, bad = 0;
  srand(12345);
  for (int trial = 0; trial < 6000; ++trial) {
    const uint32_t grid = (trial % 3 == 0) ? 512 : ((trial % 3 == 1) ? 256 : 608), one_each = grid / 2;
    const uint32_t B = 1 + rand() % ((trial % 5 == 0) ? 400 : 40), PL = 1 + rand() % 8;
    const int kind = rand() % 4;
    std::vector<uint32_t> units(B);
    const uint32_t big = 1 + rand() % 2048;
    for (auto& u : units) u = kind == 0 ? big : (kind == 1 ? 1 + rand() % 8 : (kind == 2 ? 1 + rand() % big : ((rand() % 9 == 0) ? big : 1 + rand() % 4)));
    uint32_t total = 0, umax = 0, umin = ~0u;
    std::vector<uint32_t> prefix(B + 1, 0);
    for (uint32_t b = 0; b < B; ++b) { total += units[b]; prefix[b + 1] = total; umax = units[b] > umax ? units[b] : umax; umin = units[b] < umin ? units[b] : umin; }
    const uint32_t U = PL * total, planes = PL * B;
    const uint32_t W = balanced_workgroups(grid, one_each, U, umax, umin, planes);
    ++launches;
    if (W == 0 || W > grid || W > U) { ++bad; continue; }
    const Shares shares(W, U);
    std::set<uint32_t> slots, cslots;
    std::vector<uint32_t> pieces_of(planes, 0), first_slot(planes, 0);
    unsigned long long covered = 0;
    for (uint32_t id = 0; id < W; ++id) {
      const uint32_t w = balanced_share_of(id, W);
      if (w >= W) { ++bad; continue; }
      uint32_t x = shares.begin(w);
      const uint32_t x_end = shares.begin(w + 1);
      while (x < x_end) {
        uint32_t seq = 0;
        while (PL * prefix[seq + 1] <= x) ++seq;                       // the last b with PL prefix[b] <= x
        const uint32_t u_seq = units[seq], seq_start = PL * prefix[seq];
        const uint32_t r = x - seq_start, pl = r / u_seq;
        const uint32_t S = seq_start + pl * u_seq, E = S + u_seq, stop = x_end < E ? x_end : E;
        const uint32_t first_w = x == S ? w : shares.holder(S), last_w = stop == E ? w : shares.holder(E - 1);
        const uint32_t n_pieces = last_w - first_w + 1, piece = w - first_w, plane_id = seq * PL + pl;
        const uint32_t slot0 = balanced_slot0(first_w, plane_id);
        bad += n_pieces > kBalancedMaxPieces || piece >= n_pieces;
        bad += !slots.insert(slot0 + piece).second;                     // partial rows of no two pieces collide
        bad += slot0 + piece >= balanced_slots(grid, planes);
        if (pieces_of[plane_id] == 0) first_slot[plane_id] = slot0;
        bad += first_slot[plane_id] != slot0;                          // every piece of a plane computes the same slot0
        pieces_of[plane_id] = n_pieces;
        covered += stop - x;
        x = stop;
      }
    }
    bad += covered != U;
    for (uint32_t plane = 0; plane < planes; ++plane) {
      const uint32_t n = pieces_of[plane];
      if (n == 0) { ++bad; continue; }
      if (n == 1) continue;
      const uint32_t c0 = balanced_cluster_slot0(first_slot[plane], plane);
      for (uint32_t c = 0; c < (n + kBalancedFan - 1) / kBalancedFan; ++c) {
        bad += !cslots.insert(c0 + c).second;                           // cluster counters / cluster partials of no two planes collide
        bad += c0 + c >= balanced_cluster_slots(grid, planes);
      }
    }
  }
  printf("%llu %llu\n", launches, bad);
  return 0;
}
"""


def test_a_walked_launch_numbers_its_pieces_without_collisions(tmp_path):
    """The rounding rules of the workgroup count, the XCD order of the shares and the slot formulas of
    decode_balanced.hip, walked on the host over 6000 random launches (equal planes, many short planes,
    a few long ones among short ones): a later edit to any of them fails here, not as corrupted partial
    rows on the GPU."""
    gxx = shutil.which("g++")
    if not gxx:
        pytest.skip("no g++")
    src = tmp_path / "walk.cpp"
    src.write_text(WALK)
    exe = tmp_path / "walk"
    subprocess.run([gxx, "-O2", "-std=c++17", "-Wall", "-I", CSRC, str(src), "-o", str(exe)], check=True, timeout=300)
    launches, bad = (int(x) for x in subprocess.run([str(exe)], check=True, capture_output=True, text=True,
                                                    timeout=600).stdout.split())
    assert launches == 6000 and bad == 0
