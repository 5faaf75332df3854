// Equal shares of U units for W workgroups, and back: which workgroup holds a unit; and the
// numbering of workgroups, pieces and partial slots built on it.
// Used by decode_balanced.hip on the device; plain arithmetic, also compiled by the CPU tests.
// Share g begins at floor(g U / W): shares differ by at most one unit and the longer ones are
// spread evenly, so that when the units come in P runs of equal length and W is a multiple of
// P, every run's end is a share's end.  All 32-bit (a 64-bit division on the device is a
// subroutine of a few hundred instructions): g U / W = g a + g r / W with U = a W + r, which
// needs g r < 2^32, i.e. W < 2^16; and g a <= U < 2^31.
#pragma once

#include <stdint.h>

#ifdef __HIPCC__
#define ELLM_SHARES_FN __host__ __device__ __forceinline__
#else
#define ELLM_SHARES_FN inline
#endif

namespace ellm {

struct Shares {
  uint32_t W, U, a, r;
  double w_over_u;
  ELLM_SHARES_FN Shares(uint32_t workgroups, uint32_t units)
      : W(workgroups), U(units), a(units / workgroups), r(units - (units / workgroups) * workgroups),
        w_over_u((double)workgroups / (double)units) {}
  ELLM_SHARES_FN uint32_t begin(uint32_t g) const { return g * a + g * r / W; }
  // The last g with begin(g) <= unit, i.e. ceil((unit + 1) W / U) - 1: from a double-precision
  // product that is off by at most one, corrected either way.
  ELLM_SHARES_FN uint32_t holder(uint32_t unit) const {
    uint32_t g = (uint32_t)(((double)unit + 1.0) * w_over_u);
    if (g > W - 1) g = W - 1;
    if (begin(g) > unit)
      --g;
    else if (g + 1 < W && begin(g + 1) <= unit)
      ++g;
    return g;
  }
};

// ---- how decode_balanced.hip numbers its workgroups, pieces and partial slots ----------------
// (host-compilable so that the CPU tests can walk a launch: the distinctness of the slots below
// is all that keeps partial rows and arrival counters of different planes apart)

constexpr uint32_t kBalancedFan = 16;                          // partials folded per step (decode_common.hpp: kMergeFan)
constexpr uint32_t kBalancedMaxPieces = kBalancedFan * kBalancedFan;   // two fold levels

// Units a share must at least hold so that no plane is cut into more pieces than two fold
// levels take: a plane of u units has at most u / q + 2 pieces when q = floor(U / W) units is the
// smaller share.
ELLM_SHARES_FN uint32_t balanced_min_share(uint32_t longest_plane_units) {
  return (longest_plane_units + kBalancedMaxPieces - 3) / (kBalancedMaxPieces - 2);
}
// Workgroups that take part out of `limit`: at most one per unit of work and few enough for
// balanced_min_share; with planes of equal length a whole number per plane (so that shares end
// where planes end), else a multiple of eight (one contiguous eighth of the shares per XCD).
ELLM_SHARES_FN uint32_t balanced_takers(uint32_t limit, uint32_t U, uint32_t min_share, bool equal_planes,
                                        uint32_t planes) {
  uint32_t n = limit < U ? limit : U;
  const uint32_t cap = U / min_share;
  if (cap < n) n = cap;
  if (equal_planes && planes <= n)
    n -= n % planes;
  else if (n >= 8)
    n &= ~7u;
  return n;
}
// One workgroup per compute unit (`one_each` of them) where the planes are at most as many as the
// units and that count is at least 0.47 of what the whole launch would field, else all of it.
ELLM_SHARES_FN uint32_t balanced_workgroups(uint32_t launched, uint32_t one_each, uint32_t U, uint32_t umax,
                                            uint32_t umin, uint32_t planes) {
  const uint32_t q = balanced_min_share(umax);
  uint32_t W = balanced_takers(launched, U, q, umax == umin, planes);
  if (one_each < launched && planes <= one_each) {
    const uint32_t fewer = balanced_takers(one_each, U, q, umax == umin, planes);
    if (100u * fewer >= 47u * W) W = fewer;
  }
  return W;
}
// The share workgroup `id` takes: each XCD (id % 8) one contiguous eighth when W allows.
ELLM_SHARES_FN uint32_t balanced_share_of(uint32_t id, uint32_t W) {
  return (W & 7u) == 0 ? (id & 7u) * (W >> 3) + (id >> 3) : id;
}
// Partial slot of piece `piece` of a plane whose first piece lies in share `first_share`: the pair
// (share, plane) moves on by one in exactly one of the two from piece to piece of a launch, so
// share + plane numbers the pieces without collisions.  Cluster slot of the plane's cluster c:
// plane + slot0 / 16 + c (distinct because 1 + floor(n / 16) >= ceil(n / 16)).
ELLM_SHARES_FN uint32_t balanced_slot0(uint32_t first_share, uint32_t plane) { return first_share + plane; }
ELLM_SHARES_FN uint32_t balanced_cluster_slot0(uint32_t slot0, uint32_t plane) { return plane + slot0 / kBalancedFan; }
// Sizes that hold every launch of `wgs` workgroups over `planes` planes (decode_balanced_takes).
ELLM_SHARES_FN uint32_t balanced_slots(uint32_t wgs, uint32_t planes) { return wgs + planes; }
ELLM_SHARES_FN uint32_t balanced_cluster_slots(uint32_t wgs, uint32_t planes) {
  return planes + (wgs + planes) / kBalancedFan + 2;
}

}  // namespace ellm
