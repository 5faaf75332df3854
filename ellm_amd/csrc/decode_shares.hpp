// Equal shares of U units for W workgroups, and back: which workgroup holds a unit.
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

}  // namespace ellm
