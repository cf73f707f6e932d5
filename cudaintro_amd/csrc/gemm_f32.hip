// fp32 GEMM on the gfx950 matrix cores (v_mfma_f32_32x32x2_f32: fp32 products, fp32
// accumulation): the shared LDS-tiled MFMA kernel with the fp32 fragment plumbing, plain or
// with the linear layer's bias + activation epilogue; or, when 256-column tiles would leave
// most of the chip idle or N is too ragged for them, the 32x32 k-split kernel.
#include "epilogues.h"
#include "mfma_tile.h"

namespace cig {

static bool f32_tile_ok(int64_t M, int64_t N, int64_t K, const float* A, int64_t lda,
                        const float* B, int64_t ldb, const float* C, int64_t ldc,
                        const BiasAct* ba) {
  return tile::tile_shape_ok(M, N, K, 4, A, lda, B, ldb, true) && ldc % 4 == 0 &&
         ((uintptr_t)C & 15) == 0 && !(ba && ba->bias && ((uintptr_t)ba->bias & 15));
}

bool launch_f32_mfma(cigemmContext* ctx, int64_t M, int64_t N, int64_t K, const float* A,
                     int64_t lda, const float* B, int64_t ldb, float* C, int64_t ldc,
                     const BiasAct* ba) {
  const bool tile_ok = f32_tile_ok(M, N, K, A, lda, B, ldb, C, ldc, ba);
  if (f32_small_shape_ok(M, N, K, A, lda)) {
    // Both costs in units of a quarter of one 256x256 tile's time per unit of k: the tile
    // plan's own figure against 0.115 per resident round of 32x32 tiles (2048^3: tile kernel
    // 157 us, small kernel 225 us; 1024^3: 74 us against 33 us; 512^3: 38 us against 8 us).
    const int cus = ctx->num_cus > 0 ? ctx->num_cus : 256;
    double tile_cost = 0;
    tile::best_mt(M, N, cus, &tile_cost);
    const double tiles32 = (double)((M + 31) / 32) * (double)((N + 31) / 32);
    const double small_cost = 0.115 * (tiles32 > cus ? tiles32 / cus : 1.0);
    // With a long K the tile kernel wins whenever its tiles fit one round: it can split K over
    // the idle compute units (512 x 512 x 4096: 33 us against 55 us; 1024^3: 31 against 32;
    // 512^3: 17 against 9; 960 x 3584 x 3584: 222 against 298).
    const bool one_round = ((M + 255) / 256) * ((N + tile::BN - 1) / tile::BN) <= cus;
    const bool long_k_split = tile_ok && K >= 2048 && one_round;
    // What the tile kernel cannot take (B or C rows not 16-byte aligned, an odd N) and fills the
    // chip with 128 x 128 tiles is left to the any-shape matrix-core kernel (4096 x 4095 x 4096:
    // 109 against 63 TFLOP/s; at 1000^3, 64 such tiles, this kernel is 3x the faster one).
    const double tiles128 = (double)((M + 127) / 128) * (double)((N + 127) / 128);
    if (!tile_ok && tiles128 >= cus) return false;
    if (!tile_ok || (small_cost < tile_cost && !long_k_split)) {
      launch_f32_small(ctx, M, N, K, A, lda, B, ldb, C, ldc, ba);
      return true;
    }
  }
  return tile_ok && launch_f32_tile(ctx, M, N, K, A, lda, B, ldb, C, ldc, ba);
}

bool launch_f32_tile(cigemmContext* ctx, int64_t M, int64_t N, int64_t K, const float* A,
                     int64_t lda, const float* B, int64_t ldb, float* C, int64_t ldc,
                     const BiasAct* ba) {
  if (!f32_tile_ok(M, N, K, A, lda, B, ldb, C, ldc, ba)) return false;
  if (!ba) {
    const bool split = tile::launch_tile<tile::MathF32, tile::B_KN32>(
        ctx, M, N, K * 4, A, lda * 4, B, ldb * 4, EpiStoreF32x4{C, ldc});
    set_tile_kernel_name(ctx, "f32", 16, "", split);
    return true;
  }
  bool split = false;
#define CIG_BA(HB, RL)                                                                          \
  split = tile::launch_tile<tile::MathF32, tile::B_KN32>(ctx, M, N, K * 4, A, lda * 4, B, ldb * 4, \
                                                         EpiBiasActF32x4<HB, RL>{C, ldc, ba->bias})
  if (ba->bias) {
    if (ba->relu) CIG_BA(true, true); else CIG_BA(true, false);
  } else {
    if (ba->relu) CIG_BA(false, true); else CIG_BA(false, false);
  }
#undef CIG_BA
  set_tile_kernel_name(ctx, "f32", 16, "_bias_act", split);
  return true;
}

}  // namespace cig
