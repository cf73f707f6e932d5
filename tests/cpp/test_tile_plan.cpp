// Host-only checks of the tile kernel's launch planning (csrc/tile_plan.h).
//   test_tile_plan            runs the invariants and prints "tile plan OK"
//   test_tile_plan plan       reads "kind M N K" lines (kind: bf16, f16, i8nk, i8kn, f32; K in
//                             elements) and prints "tile_rows k_ranges" for each, as the
//                             library plans them on 256 compute units with its 64 MiB of
//                             partial sums
#include <cstdio>
#include <cstdlib>
#include <cstring>

#include "tile_plan.h"

using namespace cig::tile;

static int failures = 0;
#define CHECK(cond, ...)                   \
  do {                                     \
    if (!(cond)) {                         \
      std::printf("FAILED %s: ", #cond);   \
      std::printf(__VA_ARGS__);            \
      std::printf("\n");                   \
      ++failures;                          \
    }                                      \
  } while (0)

struct Kind {
  const char* name;
  int elem, out_bytes;
  StageCost sc;
};
static const Kind kinds[] = {{"bf16", 2, 2, STAGE_COST_KN16}, {"f16", 2, 2, STAGE_COST_KN16},
                             {"i8nk", 1, 4, STAGE_COST_NK8},  {"i8kn", 1, 4, STAGE_COST_KN8},
                             {"f32", 4, 4, STAGE_COST_KN32}};

static void check_k_ranges() {
  for (int64_t K_bytes = 16; K_bytes <= 70000; K_bytes += (K_bytes < 2048 ? 16 : 1008)) {
    const int64_t kts = (K_bytes + KB - 1) / KB;
    for (int wanted = 1; wanted <= 40; ++wanted) {
      int64_t rs = 0;
      const int sp = k_ranges(K_bytes, wanted, &rs);
      CHECK(sp >= 1 && sp <= (wanted > 1 ? wanted : 1), "K %lld wanted %d -> %d", (long long)K_bytes,
            wanted, sp);
      CHECK(rs >= 1 && sp * rs >= kts && (sp - 1) * rs < kts, "K %lld wanted %d: %d x %lld stages",
            (long long)K_bytes, wanted, sp, (long long)rs);
      if (sp > 1) CHECK(rs % 2 == 0, "K %lld wanted %d: odd range %lld", (long long)K_bytes, wanted, (long long)rs);
      int64_t rs2 = 0;
      const int sp2 = k_ranges(K_bytes, sp, &rs2);  // the launcher recomputes from the count
      CHECK(sp2 == sp && rs2 == rs, "K %lld: %d ranges of %lld, again %d of %lld", (long long)K_bytes,
            sp, (long long)rs, sp2, (long long)rs2);
    }
  }
}

static void check_plans() {
  const size_t room = (size_t)64 << 20;
  for (const Kind& k : kinds)
    for (int64_t M : {1, 33, 64, 65, 100, 128, 129, 192, 256, 300, 512, 777, 1024, 2048, 4096})
      for (int64_t N : {256, 1000, 2048, 4096, 5120, 8192, 11008, 14336, 28672})
        for (int64_t K : {64, 512, 1024, 2048, 4096, 4128, 8192, 11008, 28672}) {
          if (((M + BM - 1) / BM) * ((N + BN - 1) / BN) > 256) continue;  // not plan_small's
          const int64_t K_bytes = K * k.elem;
          const SmallPlan p = plan_small(256, room, M, N, K_bytes, k.out_bytes, k.sc, K_bytes * N);
          CHECK(p.mt >= 1 && p.mt <= 4 && p.splits >= 1, "%s %lld %lld %lld: %d x %d", k.name,
                (long long)M, (long long)N, (long long)K, p.mt, p.splits);
          CHECK(p.mt == 1 || 64 * (p.mt - 1) < M, "%s M %lld: tile of %d rows", k.name, (long long)M,
                64 * p.mt);
          int64_t rs = 0;
          CHECK(k_ranges(K_bytes, p.splits, &rs) == p.splits, "%s K %lld: %d ranges", k.name,
                (long long)K, p.splits);
          if (p.splits > 1) {
            const int64_t tiles = ((M + 64 * p.mt - 1) / (64 * p.mt)) * ((N + BN - 1) / BN);
            CHECK(rs >= PlanCost::MIN_RANGE_STAGES, "%s K %lld: ranges of %lld stages", k.name,
                  (long long)K, (long long)rs);
            CHECK((size_t)p.splits * M * N * 4 <= room, "%s %lld %lld: %d ranges over the workspace",
                  k.name, (long long)M, (long long)N, p.splits);
            CHECK(tiles * p.splits <= (int64_t)PlanCost::MAX_ROUNDS_SPLIT * 256, "%s: %lld workgroups",
                  k.name, (long long)(tiles * p.splits));
          }
          // without a workspace no plan splits
          const SmallPlan q = plan_small(256, 0, M, N, K_bytes, k.out_bytes, k.sc, K_bytes * N);
          CHECK(q.splits == 1, "%s %lld %lld %lld: %d ranges without a workspace", k.name,
                (long long)M, (long long)N, (long long)K, q.splits);
        }
  // tile heights of plans of several rounds
  CHECK(best_mt(8192, 8192, 256) == 4, "8192^2: %d", best_mt(8192, 8192, 256));
  CHECK(best_mt(2048, 11008, 256) == 3, "2048 x 11008: %d", best_mt(2048, 11008, 256));
  // fp32 pays by the row: short tiles where they waste fewer rounds
  CHECK(best_mt(5120, 4096, 256, nullptr, TILE_UNITS_F32) == 1, "fp32 5120 x 4096");
  CHECK(best_mt(8192, 6144, 256, nullptr, TILE_UNITS_F32) == 4, "fp32 8192 x 6144");
  CHECK(best_mt(4096, 4096, 256, nullptr, TILE_UNITS_F32) == 4, "fp32 4096 x 4096");
}

int main(int argc, char** argv) {
  if (argc > 1 && !std::strcmp(argv[1], "plan")) {
    char kind[16];
    long long M, N, K;
    while (std::scanf("%15s %lld %lld %lld", kind, &M, &N, &K) == 4) {
      const Kind* k = nullptr;
      for (const Kind& c : kinds)
        if (!std::strcmp(c.name, kind)) k = &c;
      if (!k) {
        std::printf("0 0\n");
        continue;
      }
      const SmallPlan p = plan_small(256, (size_t)64 << 20, M, N, K * k->elem, k->out_bytes, k->sc,
                                     K * k->elem * N);
      std::printf("%d %d\n", 64 * p.mt, p.splits);
    }
    return 0;
  }
  check_k_ranges();
  check_plans();
  if (failures) {
    std::printf("%d failure(s)\n", failures);
    return 1;
  }
  std::printf("tile plan OK\n");
  return 0;
}
