"""The key-range split planner of the chunk kernels (ellm_amd/csrc/chunk_plan.hpp, host code) against an
exact simulation of the dispatch it models: workgroups dealt in id order to the free slot that
opens first."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "ellm_amd", "csrc")

PROBE = r"""
#include "chunk_plan.hpp"
#include <algorithm>
#include <cstdio>
#include <vector>
using namespace ellm;
static uint64_t simulate(uint32_t items, uint32_t slots, uint32_t len, uint32_t n, uint32_t rest) {
  std::vector<uint64_t> free_at(slots, 0);
  uint64_t end = 0;
  for (uint32_t s = 0; s < n; ++s)
    for (uint32_t i = 0; i < items; ++i) {
      auto it = std::min_element(free_at.begin(), free_at.end());
      *it += (s == n - 1) ? rest : len;
      end = std::max(end, *it);
    }
  return end;
}
int main() {
  const uint32_t tiles_set[] = {1, 7, 16, 17, 33, 64, 129, 130, 513, 2048};
  const uint32_t items_set[] = {1, 4, 8, 16, 24, 96, 128, 192, 255, 256, 300};
  const uint32_t slots_set[] = {256, 512};
  const uint32_t max_set[] = {1, 2, 5, 64, 4096};
  const double cost_set[] = {0.0, 0.1, 1.0, 6.7};
  for (uint32_t tiles : tiles_set) for (uint32_t items : items_set) for (uint32_t slots : slots_set)
  for (uint32_t max_split : max_set) for (double cost : cost_set) for (uint32_t min_tiles : {4u, 8u}) {
    const KeySplit k = plan_key_split(tiles, items, slots, min_tiles, max_split, cost);
    const uint32_t rest = tiles - (k.n_split - 1) * k.split_tiles;
    const KeySplit again = plan_key_split(tiles, items, slots, min_tiles, max_split, cost);
    printf("%u %u %u %u %u %g %u %u %u %llu %llu %llu %u %u\n", tiles, items, slots, min_tiles, max_split, cost,
           k.split_tiles, k.n_split, rest,
           (unsigned long long)key_split_makespan(items, slots, k.split_tiles, k.n_split, rest),
           (unsigned long long)simulate(items, slots, k.split_tiles, k.n_split, rest),
           (unsigned long long)simulate(items, slots, tiles, 1, tiles), again.split_tiles, again.n_split);
  }
  return 0;
}
"""


@pytest.fixture(scope="module")
def rows(tmp_path_factory):
    gxx = shutil.which("g++")
    if not gxx:
        pytest.skip("no g++")
    d = tmp_path_factory.mktemp("plan")
    src = d / "probe.cpp"
    src.write_text(PROBE)
    exe = d / "probe"
    subprocess.run([gxx, "-O2", "-std=c++17", "-I", CSRC, str(src), "-o", str(exe)], check=True, timeout=300)
    out = subprocess.run([str(exe)], check=True, capture_output=True, text=True, timeout=300).stdout
    return [[float(x) for x in line.split()] for line in out.splitlines()]


def test_plans_are_well_formed(rows):
    assert len(rows) > 1000
    for tiles, items, slots, min_tiles, max_split, cost, length, n, rest, est, sim, unsplit, l2, n2 in rows:
        assert 1 <= n <= max(max_split, 1)
        assert (n - 1) * length + rest == tiles and 1 <= rest <= length     # the pieces tile the walk, the last is the short one
        assert n == 1 or length >= min_tiles
        assert (l2, n2) == (length, n)                                       # the memo returns the same answer


def test_estimate_never_undershoots_the_simulated_dispatch_by_much(rows):
    """The closed form is what the planner minimises; it must track the simulation: never below it
    (it would pick plans that look better than they are) beyond one short piece, and within one long
    piece above."""
    for tiles, items, slots, min_tiles, max_split, cost, length, n, rest, est, sim, unsplit, l2, n2 in rows:
        assert est + rest >= sim, (tiles, items, slots, length, n, est, sim)
        assert est <= sim + length, (tiles, items, slots, length, n, est, sim)


def test_a_split_is_only_chosen_when_it_pays(rows):
    for tiles, items, slots, min_tiles, max_split, cost, length, n, rest, est, sim, unsplit, l2, n2 in rows:
        if n > 1:
            assert est + n * cost < unsplit, (tiles, items, slots, cost, length, n, est, unsplit)


def test_known_shapes(rows):
    """24 sequences x 4 kv heads on 8192 keys (129 tiles): the twelve-wave kernel (one workgroup a unit)
    gets two long pieces and a short one per plane; with twice the slots the plan is five equal pieces."""
    by = {(r[0], r[1], r[2], r[3], r[4], r[5]): r for r in rows}
    r = by[(129, 96, 256, 4, 5, 1.0)]
    assert (r[6], r[7], r[8]) == (52, 3, 25) and r[10] == 52
    r = by[(129, 96, 512, 4, 64, 1.0)]
    assert (r[6], r[7]) == (26, 5)
