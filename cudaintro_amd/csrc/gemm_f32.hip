// fp32 GEMM on the gfx950 matrix cores (v_mfma_f32_32x32x2_f32: fp32 products, fp32
// accumulation): the shared LDS-tiled MFMA kernel with the fp32 fragment plumbing, plain or
// with the linear layer's bias + activation epilogue.
#include "epilogues.h"
#include "mfma_tile.h"

namespace cig {

bool launch_f32_mfma(cigemmContext* ctx, int64_t M, int64_t N, int64_t K, const float* A,
                     int64_t lda, const float* B, int64_t ldb, float* C, int64_t ldc,
                     const BiasAct* ba) {
  if (!tile::tile_shape_ok(M, N, K, 4, A, lda, B, ldb, true)) return false;
  if (ldc % 4 || ((uintptr_t)C & 15)) return false;
  if (!ba) {
    tile::launch_tile<tile::MathF32, tile::B_KN32>(ctx, M, N, K * 4, A, lda * 4, B, ldb * 4,
                                                   EpiStoreF32x4{C, ldc});
    ctx->last_kernel = "f32_mfma_256x256x16_ring4";
    return true;
  }
  if (ba->bias && ((uintptr_t)ba->bias & 15)) return false;
#define CIG_BA(HB, RL)                                                                  \
  tile::launch_tile<tile::MathF32, tile::B_KN32>(ctx, M, N, K * 4, A, lda * 4, B, ldb * 4, \
                                                 EpiBiasActF32x4<HB, RL>{C, ldc, ba->bias})
  if (ba->bias) {
    if (ba->relu) CIG_BA(true, true); else CIG_BA(true, false);
  } else {
    if (ba->relu) CIG_BA(false, true); else CIG_BA(false, false);
  }
#undef CIG_BA
  ctx->last_kernel = "f32_mfma_256x256x16_ring4_bias_act";
  return true;
}

}  // namespace cig
