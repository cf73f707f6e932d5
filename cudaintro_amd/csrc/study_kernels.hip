// Study kernels: small, readable counterparts of the tuned GEMMs, following the reference's
// TileProgramming demo.
//
//  * matrixMulTiled: one 32x32 output tile per 1024-lane workgroup, A and B tiles staged in
//    LDS, one accumulator per lane (TileProgramming/kernel.cu:54-102 and the any-width
//    variant matmulTensor.cu:99-125).  Products and sums are rounded separately in ascending
//    k, so the result equals the reference CPU loop (tensor_utils.cu:34-45) bit for bit.
//  * matrixMulMatrixCores: one wavefront per 32x32 output tile, one
//    v_mfma_f32_32x32x16_{f16,bf16} per 16 k, operands fetched straight from global memory,
//    fp32 result (the role of matmulTensor.cu:31-68; row-major A and B, one wave per tile).
//
// The matrix-core instruction computes D = A.B + C for a 32x16 A and a 16x32 B held across
// the 64 lanes of a wave: lane l supplies A[l % 32][8 (l / 32) .. + 7] and
// B[8 (l / 32) .. + 7][l % 32], and receives D[8 q + 4 (l / 32) + e][l % 32] in element
// 4 q + e of its 16 accumulators.
#include "common.h"

namespace cig {
namespace {

constexpr int TW = 32;

__global__ __launch_bounds__(TW* TW) void matrix_mul_tiled_kernel(float* __restrict__ C,
                                                                 const float* __restrict__ A,
                                                                 const float* __restrict__ B,
                                                                 int width) {
  __shared__ float sA[TW][TW];
  __shared__ float sB[TW][TW];
  const int tx = threadIdx.x, ty = threadIdx.y;
  const int row = blockIdx.y * TW + ty, col = blockIdx.x * TW + tx;
  float sum = 0.0f;
  for (int t0 = 0; t0 < width; t0 += TW) {
    sA[ty][tx] = (row < width && t0 + tx < width) ? A[(int64_t)row * width + t0 + tx] : 0.0f;
    sB[ty][tx] = (col < width && t0 + ty < width) ? B[(int64_t)(t0 + ty) * width + col] : 0.0f;
    __syncthreads();
    // Zero padding past the edge adds +-0 to a sum that started at +0: no effect.
#pragma unroll
    for (int k = 0; k < TW; ++k) sum = __fadd_rn(sum, __fmul_rn(sA[ty][k], sB[k][tx]));
    __syncthreads();
  }
  if (row < width && col < width) C[(int64_t)row * width + col] = sum;
}

template <typename E16>
__global__ __launch_bounds__(64) void matrix_mul_mfma_kernel(const uint16_t* __restrict__ A,
                                                             const uint16_t* __restrict__ B,
                                                             float* __restrict__ C, int width) {
  const int l = threadIdx.x;
  const int r = l & 31, h = l >> 5;
  const int row = blockIdx.y * 32 + r;  // this lane's row of A
  const int col = blockIdx.x * 32 + r;  // this lane's column of B
  f32x16 acc;
#pragma unroll
  for (int i = 0; i < 16; ++i) acc[i] = 0.0f;
  for (int k0 = 0; k0 < width; k0 += 16) {
    i16x8 a, b;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int k = k0 + 8 * h + i;
      const bool in = k < width;
      a[i] = (in && row < width) ? (short)A[(int64_t)row * width + k] : (short)0;
      b[i] = (in && col < width) ? (short)B[(int64_t)k * width + col] : (short)0;
    }
    acc = E16::mfma(a, b, acc);
  }
#pragma unroll
  for (int q = 0; q < 4; ++q)
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int orow = blockIdx.y * 32 + 8 * q + 4 * h + e;
      if (orow < width && col < width) C[(int64_t)orow * width + col] = acc[4 * q + e];
    }
}

struct MfmaF16 {
  static __device__ __forceinline__ f32x16 mfma(i16x8 a, i16x8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a),
                                                  __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
};
struct MfmaBF16 {
  static __device__ __forceinline__ f32x16 mfma(i16x8 a, i16x8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a),
                                                   __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
};

cigemmStatus_t study_args(cigemmHandle_t h, const char* name, const void* A, const void* B,
                          const void* C, int width) {
  if (!h || h->magic != kCtxMagic) return CIGEMM_STATUS_NOT_INITIALIZED;
  if (width < 0) return fail(h, CIGEMM_STATUS_INVALID_VALUE, "%s: width %d < 0", name, width);
  if (width > 0 && (!A || !B || !C))
    return fail(h, CIGEMM_STATUS_INVALID_VALUE, "%s: null matrix pointer", name);
  if ((int64_t)((width + 31) / 32) > 65535)
    return fail(h, CIGEMM_STATUS_NOT_SUPPORTED, "%s: width %d needs more than 65535 tile rows",
                name, width);
  return CIGEMM_STATUS_SUCCESS;
}

}  // namespace
}  // namespace cig

using namespace cig;

extern "C" {

cigemmStatus_t cigemm_matrixMulTiled(cigemmHandle_t h, float* C, const float* A, const float* B,
                                     int width) {
  cigemmStatus_t st = study_args(h, "cigemm_matrixMulTiled", A, B, C, width);
  if (st != CIGEMM_STATUS_SUCCESS || width == 0) return st;
  const unsigned tiles = (unsigned)((width + TW - 1) / TW);
  hipLaunchKernelGGL(matrix_mul_tiled_kernel, dim3(tiles, tiles), dim3(TW, TW), 0, h->stream, C, A,
                     B, width);
  h->last_kernel = "study_tiled_f32_32x32";
  return check_launch(h, "cigemm_matrixMulTiled");
}

cigemmStatus_t cigemm_matrixMulMatrixCores(cigemmHandle_t h, const uint16_t* A, const uint16_t* B,
                                           float* C, int width) {
  cigemmStatus_t st = study_args(h, "cigemm_matrixMulMatrixCores", A, B, C, width);
  if (st != CIGEMM_STATUS_SUCCESS || width == 0) return st;
  const unsigned tiles = (unsigned)((width + 31) / 32);
  hipLaunchKernelGGL(matrix_mul_mfma_kernel<MfmaF16>, dim3(tiles, tiles), dim3(64), 0, h->stream,
                     A, B, C, width);
  h->last_kernel = "study_mfma_f16_32x32x16";
  return check_launch(h, "cigemm_matrixMulMatrixCores");
}

cigemmStatus_t cigemm_matrixMulMatrixCoresBfloat16(cigemmHandle_t h, const uint16_t* A,
                                                   const uint16_t* B, float* C, int width) {
  cigemmStatus_t st = study_args(h, "cigemm_matrixMulMatrixCoresBfloat16", A, B, C, width);
  if (st != CIGEMM_STATUS_SUCCESS || width == 0) return st;
  const unsigned tiles = (unsigned)((width + 31) / 32);
  hipLaunchKernelGGL(matrix_mul_mfma_kernel<MfmaBF16>, dim3(tiles, tiles), dim3(64), 0, h->stream,
                     A, B, C, width);
  h->last_kernel = "study_mfma_bf16_32x32x16";
  return check_launch(h, "cigemm_matrixMulMatrixCoresBfloat16");
}

}  // extern "C"
