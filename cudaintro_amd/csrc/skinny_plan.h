// Launch planning of the K-over-the-waves decode kernel (gemm_skinny.hip), as plain host
// functions of sizes so that a host-only test can check them.
#pragma once
#include <cstddef>
#include <cstdint>

namespace cig {
namespace skinny_plan {

// K ranges per slab, up to 16, each of at least 8 stages, partials (128 bytes per column, slab
// and range: 32 rows of 4-byte sums) and counters (4 bytes per slab) within the workspace.  Two
// workgroups fit a compute unit, and the ones that share a unit share its rate: a launch takes
// about (stages per range) x (workgroups on the fullest unit), so that is what the count
// minimises; more ranges are taken only when they make it a tenth smaller (their exchange
// costs, too).  N = K = 8192 in 128-column slabs: 64 slabs x 4 ranges = one workgroup per unit.
// N = 11008, K = 4096: 86 slabs x 5 = 430 workgroups, two on most units (20.4 us; 4 ranges, two
// on a third of the units, 22.3; 2 ranges, 172 units busy, 20.9; 3 ranges 23.8).  N = 13824,
// K = 5120: 108 slabs x 2.
inline int kwaves_splits(int64_t slabs, int64_t stages, int cols, int cus, size_t counter_bytes,
                         size_t partial_bytes) {
  if (cus <= 0) cus = 256;
  if ((size_t)slabs * 4 > counter_bytes) return 1;
  int best = 1;
  int64_t best_cost = stages * ((slabs + cus - 1) / cus) * 16;  // in sixteenths of a stage
  for (int s = 2; s <= 16; ++s) {
    if (stages / s < 8 || slabs * s > 2 * (int64_t)cus) break;
    if ((size_t)s * (size_t)slabs * 128 * (size_t)cols > partial_bytes) break;
    const int64_t cost = (stages * 16 / s) * ((slabs * s + cus - 1) / cus);
    if (cost * 10 < best_cost * 9) {
      best_cost = cost;
      best = s;
    }
  }
  return best;
}

// The kernel with 256-column (16-bit) or 128-column (int8) slabs and a workgroup barrier per
// stage: number of K ranges, a power of two up to 16 -- enough workgroups to cover the chip
// about once, at least 4 stages per range, partials (`xrows` rows of 4-byte sums per column and
// range) and counters within the workspace.
inline int barrier_kernel_splits(int64_t slabs, int64_t N, int64_t stages, int xrows, int cus,
                                 size_t counter_bytes, size_t partial_bytes) {
  int s = 1;
  while (s < 16 && slabs * s < cus && stages % (2 * s) == 0 && stages / (2 * s) >= 4 &&
         (size_t)(2 * s) * (size_t)xrows * (size_t)N * 4 <= partial_bytes)
    s *= 2;
  if ((size_t)slabs * 4 > counter_bytes) s = 1;
  return s;
}

// int8 N x K weights in 32-row slabs, few slabs and more than `xr` rows of x: the rows are cut into
// tiles of `xr` rows (8 or 16) that get workgroups of their own, as long as every workgroup
// still finds a compute unit and the slabs come in whole groups of 8 (the block order then
// puts the tiles of a slab on one XCD, whose L2 serves the slab's weights to all but the first).
// Returns the number of tiles, 0 when that does not apply.
inline int nk8_row_tiles(int64_t M, int64_t N, int xr, int cus) {
  if (cus <= 0) cus = 256;
  const int64_t slabs = N / 32, tiles = (M + xr - 1) / xr;
  return tiles > 1 && slabs % 8 == 0 && slabs * tiles <= cus ? (int)tiles : 0;
}

// K x N weights with 33 to 64 rows of x (two 32-row tiles per wave): taken when slabs x K ranges
// put exactly one workgroup on every compute unit.
inline bool two_tiles_fit(int64_t slabs, int64_t stages, int cols, int cus, size_t counter_bytes,
                          size_t partial_bytes) {
  if (cus <= 0) cus = 256;
  return slabs * kwaves_splits(slabs, stages, cols, cus, counter_bytes, partial_bytes / 2) == cus;
}

}  // namespace skinny_plan
}  // namespace cig
