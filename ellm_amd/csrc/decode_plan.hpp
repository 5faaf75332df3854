// How the single-token kernel cuts the planes of a call into splits, and the workspace that
// holds every such plan's partial rows (host code, no device types: also compiled by the CPU
// tests).
#pragma once

#include <stddef.h>
#include <stdint.h>

namespace ellm {

// Keys handled by one workgroup step of the single-token kernel.
constexpr uint32_t kDecodeStepKeys = 64;
// Partials folded per merge step and query heads of a GQA group that one workgroup serves
// (decode_common.hpp asserts that its own constants equal these).
constexpr uint32_t kPlanMergeFan = 16;
constexpr uint32_t kPlanMaxHeadsPerGroup = 16;

struct DecodePlan {
  uint32_t split_len;
  uint32_t n_split;
};

// Sizes (in partial rows / counters) that cover every plan decode_plan() can
// return for up to batch_capacity sequences.
struct DecodeWorkspace {
  size_t rows;      // first-level partials  (x 128 and x 2 floats)
  size_t rows2;     // cluster partials      (x 128 and x 2 floats)
  size_t counters;  // uint32 arrival counters
};

inline DecodePlan decode_plan(uint32_t max_len, uint32_t batch, uint32_t n_kv_heads, uint32_t n_cu) {
  // Every plane is cut into the same number of splits.  Each workgroup has fixed costs (query
  // load, wave merge, partial write, arrival) that more, shorter workgroups pay more often, and
  // one workgroup alone on a compute unit streams a little faster than each of two that share
  // it, so one workgroup per unit is the first choice (measured against two per unit: 16 x 8192
  // keys 45.5 against 46.4 us, 1 x 131072 46.4 against 48.1, 4 x 32768 44.8 against 47.8,
  // 64 x 2048 42.8 against 46.6).  Where the planes do not divide the units well, two per unit
  // waste less (24 x 8192: 96 planes, 2 splits = 192 workgroups on 256 units, or 5 splits = 480
  // on 2 x 256): the plan with the shorter estimated time is taken, time = keys per split x
  // workgroups on the busiest unit (x 1.03 when units are shared).  Splits are rounded down in
  // number: a few workgroups beyond a whole round make some units host one more, and those
  // finish that much later (20 x 8192: 67 us with 560 workgroups, 57 us with 480).
  const uint64_t planes = (uint64_t)batch * n_kv_heads;
  // both merge levels fold at most 16 partials: at most 16 * 16 splits per plane
  const uint32_t floor_len =
      ((max_len + kPlanMergeFan * kPlanMergeFan - 1) / (kPlanMergeFan * kPlanMergeFan) + kDecodeStepKeys - 1) /
      kDecodeStepKeys * kDecodeStepKeys;
  // Never shorter than four 64-key steps, except where even such splits leave at least half of
  // the units without a workgroup (one sequence of a few hundred keys, a handful of a thousand):
  // there a wave's chunks, fetched one after the other, are a chain of trips to memory, and one
  // 64-key step per workgroup with one fold of at most 16 partials is the shorter chain
  // (1 x 512 keys: 9.4 -> 6.7 us, 4 x 1024: 10.0 -> 8.5, 1 x 2048: 8.4; folds of at most 8 or 4
  // partials, i.e. longer splits, measured the same or slower).
  const bool tiny = planes * ((max_len + 4 * kDecodeStepKeys - 1) / (4 * kDecodeStepKeys)) * 2 <= n_cu;
  const uint32_t one_fold_len = ((max_len + kPlanMergeFan - 1) / kPlanMergeFan + kDecodeStepKeys - 1) /
                                kDecodeStepKeys * kDecodeStepKeys;
  const uint32_t min_len = tiny ? one_fold_len : 4 * kDecodeStepKeys;
  auto plan_for = [&](uint32_t per_cu, uint64_t* cost) {
    const uint32_t target = n_cu * per_cu;
    const uint32_t want = target / planes > 0 ? (uint32_t)(target / planes) : 1;
    uint32_t split_len = (max_len + want - 1) / want;
    split_len = (split_len + kDecodeStepKeys - 1) / kDecodeStepKeys * kDecodeStepKeys;
    if (split_len < min_len) split_len = min_len;
    if (split_len < floor_len) split_len = floor_len;
    DecodePlan plan;
    plan.split_len = split_len;
    plan.n_split = (max_len + split_len - 1) / split_len;
    const uint64_t on_busiest = (planes * plan.n_split + n_cu - 1) / n_cu;
    *cost = (uint64_t)split_len * on_busiest * (on_busiest > 1 ? 103 : 100);
    return plan;
  };
  uint64_t cost_one = 0, cost_two = 0;
  const DecodePlan one = plan_for(1, &cost_one), two = plan_for(2, &cost_two);
  return cost_one <= cost_two ? one : two;
}

inline DecodeWorkspace decode_workspace(uint32_t batch_capacity, uint32_t n_q_heads, uint32_t n_kv_heads,
                                 uint32_t n_cu) {
  // rows = batch * heads * n_split with n_split <= ceil(4*n_cu / (batch*kv_heads))
  const size_t group = n_q_heads / n_kv_heads;
  DecodeWorkspace w;
  w.rows = (size_t)batch_capacity * n_q_heads + (size_t)n_cu * 16 * group;
  // cluster partials: ceil(n_split / 16) per row of batch * heads
  w.rows2 = w.rows / kPlanMergeFan + (size_t)batch_capacity * n_q_heads;
  // counters: (1 + clusters) per plane, planes <= batch * heads
  w.counters = w.rows2 + (size_t)batch_capacity * n_q_heads;
  return w;
}

// Which bound of the workspace a plan exceeds: 0 none, 1 split partials, 2 cluster partials,
// 3 arrival counters.  Cluster partials are written only when a plane has more splits than one
// fold takes (n_split > kPlanMergeFan); with fewer the single fold goes straight to the output.
inline int decode_plan_exceeds(const DecodeWorkspace& w, uint32_t batch, uint32_t n_q_heads,
                               uint32_t n_kv_heads, uint32_t group, uint32_t n_split) {
  const size_t n_cluster = (n_split + kPlanMergeFan - 1) / kPlanMergeFan;
  const size_t head_groups = (group + kPlanMaxHeadsPerGroup - 1) / kPlanMaxHeadsPerGroup;
  if ((size_t)batch * n_q_heads * n_split > w.rows) return 1;
  if (n_cluster > 1 && (size_t)batch * n_q_heads * n_cluster > w.rows2) return 2;
  if ((size_t)batch * n_kv_heads * head_groups * (1 + n_cluster) > w.counters) return 3;
  return 0;
}

inline bool decode_plan_fits(const DecodeWorkspace& w, uint32_t batch, uint32_t n_q_heads,
                      uint32_t n_kv_heads, uint32_t group, uint32_t n_split) {
  return decode_plan_exceeds(w, batch, n_q_heads, n_kv_heads, group, n_split) == 0;
}

// Capacity of the static scratch of the entry point that allocates nothing (noalloc.hip), in
// the units of DecodeWorkspace.  A launch with more than one split per K/V plane has at most
// 2 x compute units workgroups, so (sequences x query heads x splits) <= group size x 2 x
// compute units partial rows: 8192 rows cover GQA groups of up to 16 query heads on a 256-unit
// part whatever the plan.  With more than 16 splits a plane the cluster partials are at most
// rows / 16 + sequences x query heads < 1024 rows; the counters are (1 + clusters) per plane.
constexpr size_t kStaticRows = 8192;       // split partials   [row][128] + [row][2] floats
constexpr size_t kStaticRows2 = 1536;      // cluster partials [row][128] + [row][2] floats
constexpr size_t kStaticCounters = 4096;   // uint32 arrival counters

}  // namespace ellm
