// Host-only checks of the decode kernel's launch planning (csrc/skinny_plan.h): invariants over a
// sweep of sizes, and the counts the measurements behind the rule were taken at.
#include <cstdio>
#include <cstdlib>
#include <initializer_list>

#include "skinny_plan.h"

using cig::skinny_plan::barrier_kernel_splits;
using cig::skinny_plan::kwaves_splits;
using cig::skinny_plan::nk8_row_tiles;
using cig::skinny_plan::two_tiles_fit;

static int failures = 0;
#define EXPECT(cond)                                                     \
  do {                                                                   \
    if (!(cond)) {                                                       \
      std::printf("FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond);      \
      ++failures;                                                        \
    }                                                                    \
  } while (0)

int main() {
  const size_t counters = 4096, partials = (size_t)64 << 20;
  // 16-bit weights: a stage is 64 k
  EXPECT(kwaves_splits(8192 / 128, 8192 / 64, 128, 256, counters, partials) == 4);
  EXPECT(kwaves_splits(11008 / 128, 4096 / 64, 128, 256, counters, partials) == 5);
  EXPECT(kwaves_splits(12288 / 128, 4096 / 64, 128, 256, counters, partials) == 5);
  EXPECT(kwaves_splits(13824 / 128, 5120 / 64, 128, 256, counters, partials) == 2);
  EXPECT(kwaves_splits(22016 / 128, 4096 / 64, 128, 256, counters, partials) == 1);
  EXPECT(kwaves_splits(28672 / 128, 8192 / 64, 128, 256, counters, partials) == 1);
  EXPECT(kwaves_splits(6144 / 128, 6144 / 64, 128, 256, counters, partials) == 5);
  EXPECT(kwaves_splits(5120 / 128, 5120 / 64, 128, 256, counters, partials) == 6);
  EXPECT(kwaves_splits(16384 / 128, 4096 / 64, 128, 256, counters, partials) == 2);
  EXPECT(kwaves_splits(4096 / 64, 4096 / 64, 64, 256, counters, partials) == 4);
  EXPECT(kwaves_splits(1024 / 64, 8192 / 64, 64, 256, counters, partials) == 16);
  EXPECT(kwaves_splits(8128 / 64, 1024 / 64, 64, 256, counters, partials) == 2);
  EXPECT(kwaves_splits(4480 / 64, 1600 / 64, 64, 256, counters, partials) == 3);
  // int8 K x N weights: a stage is 128 k
  EXPECT(kwaves_splits(11008 / 128, 4096 / 128, 128, 256, counters, partials) == 2);
  EXPECT(kwaves_splits(8192 / 128, 8192 / 128, 128, 256, counters, partials) == 4);
  // no room for counters or partials: no exchange
  EXPECT(kwaves_splits(2000, 512, 64, 256, counters, partials) == 1);
  EXPECT(kwaves_splits(64, 128, 128, 256, counters, 0) == 1);
  EXPECT(kwaves_splits(64, 128, 128, 256, counters, (size_t)3 * 64 * 128 * 128) == 3);
  // a device that does not report its units counts as 256
  EXPECT(kwaves_splits(64, 128, 128, 0, counters, partials) == 4);

  // rows of x in tiles for int8 N x K weights with few slabs
  EXPECT(nk8_row_tiles(32, 4096, 8, 256) == 0);    // 128 slabs x 4 tiles > 256 units
  EXPECT(nk8_row_tiles(32, 4096, 16, 256) == 2);
  EXPECT(nk8_row_tiles(16, 4096, 8, 256) == 2);
  EXPECT(nk8_row_tiles(8, 4096, 8, 256) == 0);     // one tile: nothing to cut
  EXPECT(nk8_row_tiles(32, 2048, 8, 256) == 4);
  EXPECT(nk8_row_tiles(20, 2048, 8, 256) == 3);
  EXPECT(nk8_row_tiles(32, 5120, 16, 256) == 0);   // 160 slabs x 2 > 256
  EXPECT(nk8_row_tiles(32, 2048 + 32, 8, 256) == 0);  // 65 slabs: not in groups of 8
  EXPECT(nk8_row_tiles(32, 2048, 8, 0) == 4);
  // 33 to 64 rows of x: exactly one workgroup per unit
  EXPECT(two_tiles_fit(4096 / 128, 4096 / 64, 128, 256, counters, partials));
  EXPECT(two_tiles_fit(8192 / 128, 8192 / 64, 128, 256, counters, partials));
  EXPECT(two_tiles_fit(16384 / 128, 4096 / 64, 128, 256, counters, partials));
  EXPECT(two_tiles_fit(32768 / 128, 2048 / 64, 128, 256, counters, partials));
  EXPECT(!two_tiles_fit(11008 / 128, 4096 / 64, 128, 256, counters, partials));
  EXPECT(!two_tiles_fit(28672 / 128, 8192 / 64, 128, 256, counters, partials));
  EXPECT(!two_tiles_fit(13824 / 128, 5120 / 64, 128, 256, counters, partials));
  EXPECT(!two_tiles_fit(5120 / 128, 5120 / 64, 128, 256, counters, partials));

  // invariants over a sweep
  long checked = 0;
  for (int cus : {32, 64, 120, 256, 304})
    for (int cols : {64, 128})
      for (int64_t slabs = 1; slabs <= 1200; slabs += (slabs < 300 ? 1 : 37))
        for (int64_t stages = 1; stages <= 600; stages += (stages < 40 ? 1 : 13)) {
          const int s = kwaves_splits(slabs, stages, cols, cus, counters, partials);
          ++checked;
          EXPECT(s >= 1 && s <= 16);
          if (s > 1) {
            EXPECT(stages / s >= 8);                 // ranges of at least 8 stages
            EXPECT(slabs * s <= 2 * (int64_t)cus);   // at most two workgroups per unit
            EXPECT((size_t)slabs * 4 <= counters);
            EXPECT((size_t)s * slabs * 128 * cols <= partials);
            // never worse than a single range by the rule's own measure
            EXPECT((stages * 16 / s) * ((slabs * s + cus - 1) / cus) <
                   stages * 16 * ((slabs + cus - 1) / cus));
          }
          if (failures > 20) return 1;
        }
  // The entry point that allocates nothing plans with a 16 MiB partial area and 4 KiB of
  // counters where a handle has 64 MiB and 64 KiB, and promises the same bits as the handle
  // entry: up to its limit of N = 16384 both must pick the same K ranges, in every kernel it
  // can dispatch to (64- and 128-column slabs of the K-over-the-waves kernel, two row tiles
  // included, and the 256-column slabs of the barrier kernel), for every K.
  for (int64_t N = 64; N <= 16384; N += 64)
    for (int64_t K = 32; K <= 32768; K += (K < 4096 ? 32 : 416)) {
      const size_t sc = 4096, sp = (size_t)16 << 20, hc = (size_t)64 << 10, hp = (size_t)64 << 20;
      for (int cols : {64, 128})
        if (N % cols == 0 && K % 64 == 0)
          for (int x_tiles : {1, 2}) {
            ++checked;
            EXPECT(kwaves_splits(N / cols, K / 64, cols, 256, sc, sp / x_tiles) ==
                   kwaves_splits(N / cols, K / 64, cols, 256, hc, hp / x_tiles));
          }
      if (N % 256 == 0) {
        ++checked;
        EXPECT(barrier_kernel_splits(N / 256, N, K / 32, 32, 256, sc, sp) ==
               barrier_kernel_splits(N / 256, N, K / 32, 32, 256, hc, hp));
      }
      if (failures > 20) return 1;
    }
  if (failures) return 1;
  std::printf("skinny plan OK (%ld cases)\n", checked);
  return 0;
}
