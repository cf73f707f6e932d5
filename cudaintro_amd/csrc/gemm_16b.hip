// fp16 / bf16 GEMM on the gfx950 matrix cores: C[MxN] = A[MxK] . B[KxN], row-major, 16-bit
// in, fp32 accumulate (v_mfma_f32_32x32x16_{f16,bf16}), one round-to-nearest-even narrowing
// out.  The kernel itself is the shared LDS-tiled MFMA kernel; this file supplies the
// 16-bit epilogue and the shape gate.
#include "epilogues.h"
#include "mfma_tile.h"

namespace cig {

bool launch_16b_mfma(cigemmContext* ctx, bool bf16, int64_t M, int64_t N, int64_t K,
                     const uint16_t* A, int64_t lda, const uint16_t* B, int64_t ldb, uint16_t* C,
                     int64_t ldc) {
  if (!tile::tile_shape_ok(M, N, K, 2, A, lda, B, ldb, true)) return false;
  if (ldc % 8 || ((uintptr_t)C & 15)) return false;  // output rows are stored in 16-byte pieces
  if (bf16) {
    const bool split = tile::launch_tile<tile::MathBF16, tile::B_KN16>(
        ctx, M, N, K * 2, A, lda * 2, B, ldb * 2, EpiStore16x4<BF16>{C, ldc});
    set_tile_kernel_name(ctx, "bf16", 32, "", split);
  } else {
    const bool split = tile::launch_tile<tile::MathF16, tile::B_KN16>(
        ctx, M, N, K * 2, A, lda * 2, B, ldb * 2, EpiStore16x4<F16>{C, ldc});
    set_tile_kernel_name(ctx, "f16", 32, "", split);
  }
  return true;
}

}  // namespace cig
