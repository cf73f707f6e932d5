// int8 GEMM on the gfx950 matrix cores (v_mfma_i32_32x32x32_i8, exact int32 accumulation)
// with either raw int32 output or the fused scale-and-dequantize epilogue.  The kernel is
// the shared LDS-tiled MFMA kernel; this file supplies the int8 epilogues and the gate.
#include "epilogues.h"
#include "mfma_tile.h"

namespace cig {
namespace {

template <int BMODE>
bool launch_layout(cigemmContext* ctx, int64_t M, int64_t N, int64_t K, const int8_t* A,
                   int64_t lda, const int8_t* B, int64_t ldb, int32_t* C, int64_t ldc,
                   const DequantArgs* dq) {
  if (!dq) {
    return tile::launch_tile<tile::MathI8, BMODE>(ctx, M, N, K, A, lda, B, ldb,
                                                  EpiStoreI32x4{C, ldc});
  }
#define CIG_DQ(OB, DA)                                                                        \
  return tile::launch_tile<tile::MathI8, BMODE>(                                              \
      ctx, M, N, K, A, lda, B, ldb,                                                           \
      EpiDequantX4<OB, DA>{dq->out, dq->ldo, dq->sa, dq->sb, dq->sa_vec, dq->sb_vec,          \
                           dq->acc_out, dq->ldacc})
  const bool dump = dq->acc_out != nullptr;
  if (dq->out_bf16) {
    if (dump) CIG_DQ(true, true); else CIG_DQ(true, false);
  } else {
    if (dump) CIG_DQ(false, true); else CIG_DQ(false, false);
  }
#undef CIG_DQ
}

}  // namespace

bool launch_i8_mfma(cigemmContext* ctx, int64_t M, int64_t N, int64_t K, const int8_t* A,
                    int64_t lda, const int8_t* B, int64_t ldb, bool b_nk, int32_t* C, int64_t ldc,
                    const DequantArgs* dq) {
  if (!tile::i8_tile_ok(M, N, K, A, lda, B, ldb, b_nk, C, ldc, dq)) return false;
  const bool split = b_nk ? launch_layout<tile::B_NK>(ctx, M, N, K, A, lda, B, ldb, C, ldc, dq)
                          : launch_layout<tile::B_KN8>(ctx, M, N, K, A, lda, B, ldb, C, ldc, dq);
  set_tile_kernel_name(ctx, "i8", 64, dq ? (b_nk ? "_nk_dequant" : "_kn_dequant") : (b_nk ? "_nk" : "_kn"),
                       split);
  return true;
}

}  // namespace cig
