// Measurement aid: one launch of the 256-row, four-wave LDS-tiled matrix-core kernel with
// timestamps taken inside every workgroup (start, first stage landed, main loop done, stores
// acknowledged), reduced on the host to the time each phase takes, the matrix-core issue cycles
// per stage and the shader clock the chip held in the main loop.  The kernel is the product
// kernel itself (same template, same schedule); only the four stamps are added.
#include <algorithm>
#include <utility>
#include <vector>

#include "cigemm_probe.h"
#include "epilogues.h"
#include "mfma_tile2.h"

namespace cig {
namespace {

template <typename Math, int BMODE, bool TWO_PER_UNIT, typename Epi, int MT = 4>
cigemmStatus_t run_profiled(cigemmContext* ctx, const char* name, int64_t M, int64_t N,
                            int64_t K_bytes, const void* A, int64_t lda_bytes, const void* B,
                            int64_t ldb_bytes, const Epi& base, double* out, int same_tile = 0) {
  constexpr int ROWS = TWO_PER_UNIT ? tile::T2_TILE_M : 64 * MT;
  const int64_t tiles = ((M + ROWS - 1) / ROWS) * ((N + tile::BN - 1) / tile::BN);
  if (!ctx->workspace || (size_t)tiles * 64 > ctx->ws_partial_bytes)
    return fail(ctx, CIGEMM_STATUS_NOT_SUPPORTED, "%s: %lld tiles exceed the workspace", name,
                (long long)tiles);
  uint64_t* stamps = static_cast<uint64_t*>(ctx->workspace);
  tile::EpiProfiled<Epi> epi{base, stamps, same_tile};
  if constexpr (TWO_PER_UNIT)
    tile::launch_tile2<Math, BMODE, tile::EpiProfiled<Epi>>(ctx, M, N, K_bytes, A, lda_bytes, B,
                                                            ldb_bytes, epi);
  else
    tile::launch_tile_mt<Math, BMODE, MT, tile::EpiProfiled<Epi>, 2>(ctx, M, N, K_bytes, A,
                                                                    lda_bytes, B, ldb_bytes, epi);
  cigemmStatus_t st = check_launch(ctx, name);
  if (st != CIGEMM_STATUS_SUCCESS) return st;
  std::vector<uint64_t> h((size_t)tiles * 8);
  if (hipMemcpyAsync(h.data(), stamps, h.size() * 8, hipMemcpyDeviceToHost, ctx->stream) != hipSuccess ||
      hipStreamSynchronize(ctx->stream) != hipSuccess) {
    (void)hipGetLastError();
    ctx->ws_dirty = 1;
    return fail(ctx, CIGEMM_STATUS_EXECUTION_FAILED, "%s: reading the stamps back failed", name);
  }
  // microseconds per tick of the constant-rate counter (100 MHz on gfx950)
  double tick_us = 0.01;
  {
    int khz = 0;
    if (hipDeviceGetAttribute(&khz, hipDeviceAttributeWallClockRate, ctx->device) == hipSuccess && khz > 0)
      tick_us = 1.0e3 / (double)khz;
    else
      (void)hipGetLastError();
  }
  const int64_t kts = (K_bytes + tile::KB - 1) / tile::KB;
  double phase_us[3] = {0, 0, 0}, main_cycles = 0, main_ticks = 0;
  uint64_t first_start = ~0ull, last_end = 0, first_epi = ~0ull, last_main_end = 0;
  for (int64_t g = 0; g < tiles; ++g) {
    const uint64_t* s = &h[(size_t)g * 8];
    for (int p = 0; p < 3; ++p) phase_us[p] += (double)(s[2 * p + 3] - s[2 * p + 1]) * tick_us;
    main_cycles += (double)(s[4] - s[2]);
    main_ticks += (double)(s[5] - s[3]);
    first_start = std::min(first_start, s[1]);
    last_end = std::max(last_end, s[7]);
    first_epi = std::min(first_epi, s[5]);
    last_main_end = std::max(last_main_end, s[5]);
  }
  out[0] = phase_us[0] / tiles;                       // start -> first stage in registers
  out[1] = phase_us[1] / tiles;                       // main loop
  out[2] = phase_us[2] / tiles;                       // epilogue, stores acknowledged
  out[3] = (double)(last_end - first_start) * tick_us;  // first workgroup start -> last end
  out[4] = main_cycles / tiles / (double)kts;         // shader cycles per 64-byte stage
  // GHz held in the main loop (0 when it is shorter than a tick of the wall clock)
  out[5] = main_ticks > 0 ? main_cycles / (main_ticks * tick_us) * 1e-3 : 0.0;
  out[6] = (double)(last_end - first_epi) * tick_us;  // first epilogue start -> last end
  out[7] = (double)tiles;
  // Per XCD (the chip's eight compute dies hold their own clocks): main-loop clock of the
  // slowest and of the fastest die; and per compute unit the end of its last workgroup, averaged
  // over the units: the launch ends with the slowest unit, `out[3]`.
  {
    double xcc_cycles[16] = {0}, xcc_ticks[16] = {0};
    std::vector<std::pair<uint64_t, uint64_t>> unit_end;  // (unit key, end of its last workgroup)
    for (int64_t g = 0; g < tiles; ++g) {
      const uint64_t* s = &h[(size_t)g * 8];
      const int xcc = (int)((s[0] >> 32) & 15);
      xcc_cycles[xcc] += (double)(s[4] - s[2]);
      xcc_ticks[xcc] += (double)(s[5] - s[3]);
      // unit = (XCC, shader engine, shader array, compute unit) of the hardware id
      const uint64_t key = ((s[0] >> 32) << 16) | ((s[0] >> 8) & 0xff);
      unit_end.emplace_back(key, s[7]);
    }
    double lo = 0, hi = 0;
    int dies = 0;
    for (int x = 0; x < 16; ++x)
      if (xcc_ticks[x] > 0) {
        const double ghz = xcc_cycles[x] / (xcc_ticks[x] * tick_us) * 1e-3;
        lo = dies ? std::min(lo, ghz) : ghz;
        hi = dies ? std::max(hi, ghz) : ghz;
        ++dies;
      }
    std::sort(unit_end.begin(), unit_end.end());
    double sum_end = 0;
    int units = 0;
    for (size_t i = 0; i < unit_end.size(); ++i)
      if (i + 1 == unit_end.size() || unit_end[i + 1].first != unit_end[i].first) {
        sum_end += (double)(unit_end[i].second - first_start) * tick_us;
        ++units;
      }
    out[8] = lo;
    out[9] = hi;
    out[10] = units ? sum_end / units : 0.0;
    out[11] = (double)units;
  }
  ctx->last_kernel = "tile_phase_probe";
  return CIGEMM_STATUS_SUCCESS;
}

}  // namespace
}  // namespace cig

using namespace cig;

extern "C" cigemmStatus_t cigemm_probe_tile_phases(cigemmHandle_t h, int kind, int64_t M,
                                                   int64_t N, int64_t K, const void* A,
                                                   int64_t lda, const void* B, int64_t ldb,
                                                   void* C, int64_t ldc, double* phases) {
  const char* name = "cigemm_probe_tile_phases";
  if (!h || h->magic != kCtxMagic) return CIGEMM_STATUS_NOT_INITIALIZED;
  // kind + 16: kinds 0, 1 and 4 with every workgroup on output tile (0, 0)
  const int same_tile = (kind == 16 || kind == 17 || kind == 20) ? 1 : 0;
  if (same_tile) kind -= 16;
  if (kind < 0 || kind > 5 || !A || !B || !C || !phases || M <= 0 || N <= 0 || K <= 0 ||
      lda < K || ldb < (kind == 5 ? K : N) || ldc < N)
    return fail(h, CIGEMM_STATUS_INVALID_VALUE, "%s: bad argument", name);
  const int elem = (kind == 1 || kind == 3 || kind == 5) ? 1 : 2;
  if (!tile::tile_shape_ok(M, N, K, elem, A, lda, B, ldb, kind != 5) || N % 8 || ldc % 8 ||
      ((uintptr_t)C & 15))
    return fail(h, CIGEMM_STATUS_NOT_SUPPORTED, "%s: shape or alignment outside the tile kernel's",
                name);
  const EpiStore16x4<BF16> e16{static_cast<uint16_t*>(C), ldc};
  const EpiStoreI32x4 e32{static_cast<int32_t*>(C), ldc};
  const EpiStore16x4<F16> e16h{static_cast<uint16_t*>(C), ldc};
  switch (kind) {
    case 5:
      return run_profiled<tile::MathI8, tile::B_NK, false, EpiStoreI32x4, 3>(h, name, M, N, K, A, lda, B,
                                                                            ldb, e32, phases);
    case 4:
      return run_profiled<tile::MathF16, tile::B_KN16, false>(h, name, M, N, K * 2, A, lda * 2, B,
                                                              ldb * 2, e16h, phases, same_tile);
    case 0:
      return run_profiled<tile::MathBF16, tile::B_KN16, false>(h, name, M, N, K * 2, A, lda * 2, B,
                                                               ldb * 2, e16, phases, same_tile);
    case 1:
      return run_profiled<tile::MathI8, tile::B_KN8, false>(h, name, M, N, K, A, lda, B, ldb, e32,
                                                            phases, same_tile);
    case 2:
      return run_profiled<tile::MathBF16, tile::B_KN16, true>(h, name, M, N, K * 2, A, lda * 2, B,
                                                              ldb * 2, e16, phases);
    default:
      return run_profiled<tile::MathI8, tile::B_KN8, true>(h, name, M, N, K, A, lda, B, ldb, e32,
                                                           phases);
  }
}
