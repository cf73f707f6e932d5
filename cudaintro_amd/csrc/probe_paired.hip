// Measurement aid: GEMM entry points on the two-workgroups-per-unit form of the tile kernel
// (mfma_tile2.h: 128-row tiles, two workgroups resident per compute unit and out of phase).
// The library never chooses this form: it issues more matrix instructions per cycle and is
// slower on a power-limited chip.  It lives here, beside the other probes, as the measured
// counterpart of the one-workgroup-per-unit kernel.
#include "cigemm_probe.h"
#include "epilogues.h"
#include "mfma_tile2.h"

namespace cig {
namespace {

bool valid(cigemmHandle_t h) { return h && h->magic == kCtxMagic; }

cigemmStatus_t check_args(cigemmHandle_t h, const char* name, int64_t M, int64_t N, int64_t K,
                          const void* A, int64_t lda, const void* B, int64_t ldb, const void* C,
                          int64_t ldc) {
  if (M <= 0 || N <= 0 || K <= 0 || !A || !B || !C || lda < K || ldb < N || ldc < N)
    return fail(h, CIGEMM_STATUS_INVALID_VALUE, "%s: bad argument", name);
  return CIGEMM_STATUS_SUCCESS;
}

cigemmStatus_t refused(cigemmHandle_t h, const char* name) {
  return fail(h, CIGEMM_STATUS_NOT_SUPPORTED,
              "%s: shape or alignment outside what the paired tile kernel takes", name);
}

cigemmStatus_t gemm16_paired(cigemmHandle_t h, const char* name, bool bf16, int64_t M, int64_t N,
                             int64_t K, const uint16_t* A, int64_t lda, const uint16_t* B,
                             int64_t ldb, uint16_t* C, int64_t ldc) {
  if (!valid(h)) return CIGEMM_STATUS_NOT_INITIALIZED;
  const cigemmStatus_t st = check_args(h, name, M, N, K, A, lda, B, ldb, C, ldc);
  if (st != CIGEMM_STATUS_SUCCESS) return st;
  if (!tile::tile_shape_ok(M, N, K, 2, A, lda, B, ldb, true) || ldc % 8 || ((uintptr_t)C & 15))
    return refused(h, name);
  h->first_tile_rows = 0;
  h->first_waves = 0;
  if (bf16)
    tile::launch_tile2<tile::MathBF16, tile::B_KN16>(h, M, N, K * 2, A, lda * 2, B, ldb * 2,
                                                     EpiStore16x4<BF16>{C, ldc});
  else
    tile::launch_tile2<tile::MathF16, tile::B_KN16>(h, M, N, K * 2, A, lda * 2, B, ldb * 2,
                                                    EpiStore16x4<F16>{C, ldc});
  set_tile_kernel_name(h, bf16 ? "bf16" : "f16", 32, "", false);
  return check_launch(h, name);
}

cigemmStatus_t gemm_i8_paired(cigemmHandle_t h, const char* name, int64_t M, int64_t N, int64_t K,
                              const int8_t* A, int64_t lda, const int8_t* B, int64_t ldb,
                              int32_t* C, int64_t ldc, const DequantArgs* dq) {
  if (!tile::i8_tile_ok(M, N, K, A, lda, B, ldb, false, C, ldc, dq)) return refused(h, name);
  h->first_tile_rows = 0;
  h->first_waves = 0;
  if (!dq) {
    tile::launch_tile2<tile::MathI8, tile::B_KN8>(h, M, N, K, A, lda, B, ldb, EpiStoreI32x4{C, ldc});
  } else {
#define CIG_DQ2(OB, DA)                                                                       \
  tile::launch_tile2<tile::MathI8, tile::B_KN8>(                                              \
      h, M, N, K, A, lda, B, ldb,                                                             \
      EpiDequantX4<OB, DA>{dq->out, dq->ldo, dq->sa, dq->sb, dq->sa_vec, dq->sb_vec,          \
                           dq->acc_out, dq->ldacc})
    const bool dump = dq->acc_out != nullptr;
    if (dq->out_bf16) {
      if (dump) CIG_DQ2(true, true); else CIG_DQ2(true, false);
    } else {
      if (dump) CIG_DQ2(false, true); else CIG_DQ2(false, false);
    }
#undef CIG_DQ2
  }
  set_tile_kernel_name(h, "i8", 64, dq ? "_kn_dequant" : "_kn", false);
  return check_launch(h, name);
}

}  // namespace
}  // namespace cig

using namespace cig;

extern "C" {

cigemmStatus_t cigemm_probe_gemm_bf16_paired(cigemmHandle_t h, int64_t M, int64_t N, int64_t K,
                                             const uint16_t* A, int64_t lda, const uint16_t* B,
                                             int64_t ldb, uint16_t* C, int64_t ldc) {
  return gemm16_paired(h, "cigemm_probe_gemm_bf16_paired", true, M, N, K, A, lda, B, ldb, C, ldc);
}

cigemmStatus_t cigemm_probe_gemm_f16_paired(cigemmHandle_t h, int64_t M, int64_t N, int64_t K,
                                            const uint16_t* A, int64_t lda, const uint16_t* B,
                                            int64_t ldb, uint16_t* C, int64_t ldc) {
  return gemm16_paired(h, "cigemm_probe_gemm_f16_paired", false, M, N, K, A, lda, B, ldb, C, ldc);
}

cigemmStatus_t cigemm_probe_gemm_i8_i32_paired(cigemmHandle_t h, int64_t M, int64_t N, int64_t K,
                                               const int8_t* A, int64_t lda, const int8_t* B,
                                               int64_t ldb, int32_t* C, int64_t ldc) {
  const char* name = "cigemm_probe_gemm_i8_i32_paired";
  if (!valid(h)) return CIGEMM_STATUS_NOT_INITIALIZED;
  const cigemmStatus_t st = check_args(h, name, M, N, K, A, lda, B, ldb, C, ldc);
  if (st != CIGEMM_STATUS_SUCCESS) return st;
  return gemm_i8_paired(h, name, M, N, K, A, lda, B, ldb, C, ldc, nullptr);
}

cigemmStatus_t cigemm_probe_gemm_i8_dequant_paired(
    cigemmHandle_t h, int64_t M, int64_t N, int64_t K, const int8_t* A, int64_t lda,
    const int8_t* B, int64_t ldb, const float* scaleA, cigemmScaleMode_t scaleA_mode,
    const float* scaleB, cigemmScaleMode_t scaleB_mode, void* out, cigemmOutType_t out_type,
    int64_t ldo, int32_t* acc_out, int64_t ldacc) {
  const char* name = "cigemm_probe_gemm_i8_dequant_paired";
  if (!valid(h)) return CIGEMM_STATUS_NOT_INITIALIZED;
  const cigemmStatus_t st = check_args(h, name, M, N, K, A, lda, B, ldb, out, ldo);
  if (st != CIGEMM_STATUS_SUCCESS) return st;
  if (!scaleA || !scaleB || (acc_out && ldacc < N) ||
      (scaleA_mode != CIGEMM_SCALE_TENSOR && scaleA_mode != CIGEMM_SCALE_VECTOR) ||
      (scaleB_mode != CIGEMM_SCALE_TENSOR && scaleB_mode != CIGEMM_SCALE_VECTOR) ||
      (out_type != CIGEMM_OUT_F32 && out_type != CIGEMM_OUT_BF16))
    return fail(h, CIGEMM_STATUS_INVALID_VALUE, "%s: bad argument", name);
  DequantArgs dq{scaleA, scaleB, scaleA_mode == CIGEMM_SCALE_VECTOR,
                 scaleB_mode == CIGEMM_SCALE_VECTOR, out, out_type == CIGEMM_OUT_BF16, ldo,
                 acc_out, ldacc};
  return gemm_i8_paired(h, name, M, N, K, A, lda, B, ldb, nullptr, 0, &dq);
}

}  // extern "C"
