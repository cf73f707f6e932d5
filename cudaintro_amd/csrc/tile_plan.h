// Launch planning of the LDS-DMA tile kernel (mfma_tile.h), as plain host functions of sizes
// so that a host-only test can check them: the K ranges of a split launch, the estimate that
// ranks (tile height, K ranges) plans, and the tile height of plans of several rounds.
#pragma once
#include <cstddef>
#include <cstdint>
#include <initializer_list>

namespace cig {
namespace tile {

constexpr int BM = 256, BN = 256;          // the largest output tile
constexpr int KB = 64;                     // bytes of k per stage, per row

// K ranges of a split-K launch: `wanted` ranges over K_bytes of k become ranges of an even
// number of whole stages (operand rows are fetched as 128-byte lines, two stages: an odd range
// would start every later one in the middle of a line), the last one holding what is left.
// Returns the number of ranges that gives (<= wanted) and the stages of each but the last.
inline int k_ranges(int64_t K_bytes, int wanted, int64_t* range_stages) {
  const int64_t kts = (K_bytes + KB - 1) / KB;
  if (wanted <= 1 || kts < 2) {
    *range_stages = kts;
    return 1;
  }
  int64_t rs = (kts + wanted - 1) / wanted;
  rs += rs & 1;
  *range_stages = rs;
  return (int)((kts + rs - 1) / rs);
}

// Plan for a problem that fits one round of 256-row tiles: tile height and number of K
// ranges, by estimated time.  The estimate has the terms that decide between such plans; its
// constants were chosen so that it ranks the plans of a timed sweep well (759 problems: batch
// sizes 33..2048 over weight shapes of common decoder layers, bf16, int8 in both layouts and
// fp32, every tile height x 1..32 ranges timed; tests/test_tile_plan.py checks the ranking
// against those timings) and, second, so that it stays near the times themselves (rms error 12 %
// on plans within 30 % of the best).  The plan it picks is 2 % slower than the best plan timed
// on average, on those problems and on 237 others first timed afterwards.
//   One round of workgroups = a fixed cost + stages per range x cost of a stage + this round's
//   share of the memory traffic (both operands once, plus the partial sums or the output,
//   weighted) at a streaming rate; a last, partly filled round is priced by its own number of
//   workgroups.
//   A split plan adds the reduction launch as measured: max(4.75, 1.1 + bytes / 5.3 TB/s) us
//   for `splits` fp32 partial matrices read and one output written.
// A stage costs a workgroup a part that does not depend on the tile height (it waits for its
// operands: with three stages in flight the wait per stage is a third of the memory latency,
// less when B sits in the L2 / Infinity Cache) plus a part per 64 rows (LDS reads and matrix
// instructions; fp32, whose matrix instructions are 16 times slower, is the one layout where
// that part dominates).
struct SmallPlan {
  int mt;
  int splits;
};
struct StageCost {
  double fixed_us;     // per 64-byte stage, whatever the tile height (B streams from HBM)
  double per_64_rows_us;
};
// by operand layout: 16-bit K x N, int8 N x K, int8 K x N, fp32 K x N
constexpr StageCost STAGE_COST_KN16{0.234, 0.032};
constexpr StageCost STAGE_COST_NK8{0.327, 0.008};
constexpr StageCost STAGE_COST_KN8{0.261, 0.037};
constexpr StageCost STAGE_COST_KN32{0.061, 0.746};
struct PlanCost {
  // (the fixed cost of a round came out near zero: what a launch costs whatever the plan does
  // not help to choose one)
  static constexpr double ROUND_US = 0.05;         // ramp and epilogue of a round of workgroups
  static constexpr double LATER_ROUND_US = 0.05;   // the same for a partly filled last round
  static constexpr double HBM_TB_S = 9.0;
  static constexpr double PARTIAL_WEIGHT = 3.43;   // bytes of partial sums / output, weighted
  static constexpr double RESIDENT_FIXED = 0.857;  // factor on StageCost::fixed_us, B <= 16 MiB
  static constexpr int MIN_RANGE_STAGES = 8;
  static constexpr int MAX_ROUNDS_SPLIT = 3;
};
inline double plan_us(int64_t M, int64_t N, int64_t K_bytes, int out_bytes, StageCost sc,
                      bool streamed, int cus, int mt, int sp, int64_t range_stages) {
  const int64_t tiles = ((M + 64 * mt - 1) / (64 * mt)) * ((N + BN - 1) / BN);
  const int64_t wgs = tiles * sp, full = wgs / cus, rem = wgs % cus;
  const double stage =
      (streamed ? sc.fixed_us : sc.fixed_us * PlanCost::RESIDENT_FIXED) + sc.per_64_rows_us * mt;
  const double mn = (double)M * (double)N;
  const double hbm_bytes = (double)(N + M) * (double)K_bytes +
                           PlanCost::PARTIAL_WEIGHT * (sp > 1 ? sp * mn * 4.0 : mn * out_bytes);
  auto round_body = [&](int64_t active) {
    return stage * (double)range_stages +
           hbm_bytes * (double)active / (double)wgs / (PlanCost::HBM_TB_S * 1e6);
  };
  double us;
  if (full > 0) {
    us = (double)full * (PlanCost::ROUND_US + round_body(cus));
    if (rem > 0) us += PlanCost::LATER_ROUND_US + round_body(rem);
  } else {
    us = PlanCost::ROUND_US + round_body(rem);
  }
  if (sp > 1) {
    const double reduce = 1.1 + (sp * 4.0 + out_bytes) * mn / 5.3e6;
    us += reduce > 4.75 ? reduce : 4.75;
  }
  return us;
}

// `partial_bytes` = room for partial sums (0: no split plans).
inline SmallPlan plan_small(int cus, size_t partial_bytes, int64_t M, int64_t N, int64_t K_bytes,
                            int out_bytes, StageCost sc, int64_t b_bytes) {
  const bool streamed = b_bytes > (16LL << 20);
  if (cus <= 0) cus = 256;
  SmallPlan best{0, 1};
  double best_us = 1e30;
  for (int mt : {4, 3, 2, 1}) {
    if (mt > 1 && 64 * (mt - 1) >= M) continue;  // the next lower height already covers M
    const int64_t tiles = ((M + 64 * mt - 1) / (64 * mt)) * ((N + BN - 1) / BN);
    int last_sp = 0;
    for (int wanted = 1; wanted <= 32; ++wanted) {
      int64_t range_stages = 0;
      const int sp = k_ranges(K_bytes, wanted, &range_stages);
      if (sp == last_sp) continue;
      last_sp = sp;
      if (sp > 1) {
        if (range_stages < PlanCost::MIN_RANGE_STAGES) break;
        if (tiles * sp > (int64_t)PlanCost::MAX_ROUNDS_SPLIT * cus) break;
        if ((size_t)sp * (size_t)M * (size_t)N * 4 > partial_bytes) break;
      }
      const double us = plan_us(M, N, K_bytes, out_bytes, sc, streamed, cus, mt, sp, range_stages);
      if (us < best_us) {
        best_us = us;
        best = SmallPlan{mt, sp};
      }
    }
  }
  return best;
}

// Cost of one tile of 64*mt rows in a plan of several rounds (compute bound), in units of a
// quarter of the 256-row tile's: a fixed part (the B panel is fetched whatever the height) plus
// a part per 64 rows.  One round of 256 tiles, N = 4096, K = 1024..4096, 16-bit and int8:
// 4.0 / 3.1-3.2 / 2.3 / 1.6-1.8.  fp32, whose matrix instructions are 16 times slower, pays
// almost by the row (TILE_UNITS_F32): 5120 x 4096 x 4096 on 64-row tiles 1179 us against 1362 on
// 192-row ones, 7000 x 4096 x 11008 4481 against 4875 on 256-row ones, 8192 x 6144 x 4096 2808
// against 2733 (there the rounds fit).
struct TileUnits {
  double fixed, per_64_rows;
};
constexpr TileUnits TILE_UNITS{0.8, 0.8};
constexpr TileUnits TILE_UNITS_F32{0.1, 0.975};
inline double tile_cost_units(int mt, TileUnits u = TILE_UNITS) {
  return u.fixed + u.per_64_rows * mt;
}

// Relative cost of covering M x N with tiles of 64*mt rows on `cus` compute units: rounds of
// workgroups times the cost of one tile; shorter tiles re-read B more often per flop.
inline double tile_plan_cost(int64_t M, int64_t N, int mt, int cus, TileUnits u = TILE_UNITS) {
  const int64_t tiles = ((M + 64 * mt - 1) / (64 * mt)) * ((N + BN - 1) / BN);
  return (double)((tiles + cus - 1) / cus) * tile_cost_units(mt, u);
}
inline int best_mt(int64_t M, int64_t N, int cus, double* cost = nullptr,
                   TileUnits u = TILE_UNITS) {
  int best = 0;
  double bc = 1e30;
  for (int mt : {4, 3, 2, 1}) {
    const double c = tile_plan_cost(M, N, mt, cus, u);
    if (c < bc) {
      bc = c;
      best = mt;
    }
  }
  if (cost) *cost = bc;
  return best;
}

}  // namespace tile
}  // namespace cig
