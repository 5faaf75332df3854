// How the chunk kernels split the key range of a call with too few query rows to fill the
// device (host code, no device types: also compiled by the CPU tests).
//
// A call has `items` independent pieces of work (row blocks of one K/V plane), each a walk
// over `tiles` key tiles.  Splitting every walk into pieces of `split_tiles` tiles (the last
// piece of a walk takes what is left) gives items x n_split workgroups, dispatched in the
// order of their linear id: every item's first piece, then every item's second piece, ...,
// so the short last pieces start last and fill the slots that the long pieces leave free.
// A piece costs its tile count; every split of a walk also costs the write and the read of
// one partial row (128 + 2 floats) per query row, `split_cost` tiles in all.
#pragma once

#include <stdint.h>

namespace ellm {

struct KeySplit {
  uint32_t split_tiles;  // tiles per piece (the last piece of a walk may be shorter)
  uint32_t n_split;      // pieces per walk
};

// Time, in tiles, until the last workgroup ends when items x n_split workgroups of
// split_tiles tiles (the last of each walk `rest` tiles) are dealt in id order to `slots`
// workgroup slots.  The long pieces run in whole rounds; the short ones share what the last,
// part-filled round of long pieces leaves free and whatever becomes free when it ends.
inline uint64_t key_split_makespan(uint32_t items, uint32_t slots, uint32_t split_tiles,
                                   uint32_t n_split, uint32_t rest) {
  const uint64_t longs = (uint64_t)items * (n_split - 1);
  const uint64_t full_rounds = longs / slots;
  const uint32_t in_last = (uint32_t)(longs % slots);  // long pieces of the part-filled round
  const uint64_t t0 = full_rounds * split_tiles;       // that round starts here
  if (in_last == 0) return t0 + (uint64_t)((items + slots - 1) / slots) * rest;
  // shorts first fill the slots - in_last free slots, round after round, until the long
  // pieces of this round end at t0 + split_tiles; what is left then has all slots
  const uint32_t free_slots = slots - in_last;
  const uint64_t rounds_before = rest ? split_tiles / rest : 0;  // whole short rounds that fit
  const uint64_t done_before = rounds_before * free_slots;
  if (done_before >= items) {
    const uint64_t rounds = ((uint64_t)items + free_slots - 1) / free_slots;
    const uint64_t shorts_end = t0 + rounds * rest;
    const uint64_t longs_end = t0 + split_tiles;
    return shorts_end > longs_end ? shorts_end : longs_end;
  }
  const uint64_t left = items - done_before;
  return t0 + split_tiles + (left + slots - 1) / slots * rest;
}

// The split with the lowest estimated time among pieces of at least min_tiles tiles and at
// most max_split pieces a walk.  split_cost: tiles' worth of time that one more piece per
// walk adds for the whole call (partial rows written and read).  Candidates per piece count
// n: equal pieces, and n - 1 long pieces L with a short rest such that r rounds of rests
// take as long as one long piece (L = tiles r / (r (n - 1) + 1), r = 1..4).
inline KeySplit plan_key_split(uint32_t tiles, uint32_t items, uint32_t slots, uint32_t min_tiles,
                               uint32_t max_split, double split_cost) {
  // (the last answer is kept: a serving loop asks the same question launch after launch)
  struct Memo {
    uint32_t tiles, items, slots, min_tiles, max_split;
    double split_cost;
    KeySplit answer;
  };
  static thread_local Memo memo = {0, 0, 0, 0, 0, 0.0, {0, 0}};
  if (memo.tiles == tiles && memo.items == items && memo.slots == slots && memo.min_tiles == min_tiles &&
      memo.max_split == max_split && memo.split_cost == split_cost && memo.answer.n_split)
    return memo.answer;
  KeySplit best = {tiles, 1};
  if (items == 0 || slots == 0 || tiles == 0) return best;
  double best_cost = (double)((items + slots - 1) / slots) * tiles;
  if (min_tiles < 1) min_tiles = 1;
  auto consider = [&](uint32_t len) {
    if (len < min_tiles || len >= tiles) return;
    const uint32_t n = (tiles + len - 1) / len;
    if (n > max_split) return;
    const uint32_t rest = tiles - (n - 1) * len;
    const double cost = (double)key_split_makespan(items, slots, len, n, rest) + n * split_cost;
    if (cost < best_cost) {
      best_cost = cost;
      best = {len, n};
    }
  };
  // more pieces than fill the slots twice over cannot pay
  const uint32_t useful = 2 * ((slots + items - 1) / items) + 2;
  const uint32_t n_max = max_split < useful ? max_split : useful;
  for (uint32_t n = 2; n <= n_max; ++n) {
    consider((tiles + n - 1) / n);
    for (uint32_t r = 1; r <= 4; ++r) {
      const uint32_t den = r * (n - 1) + 1;
      consider((uint32_t)(((uint64_t)tiles * r + den - 1) / den));
    }
  }
  memo = {tiles, items, slots, min_tiles, max_split, split_cost, best};
  return best;
}

}  // namespace ellm
