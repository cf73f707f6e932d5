// Any-shape GEMM kernels: the path for sizes, leading dimensions or pointer alignments the
// MFMA families do not take (ragged tails, M/N/K of 1, odd ld).  One 64x64 output tile per
// 256-thread workgroup, 16-deep LDS slabs, a 4x4 register block per lane, every load and
// store bounds-checked.  Arithmetic is scalar VALU:
//   - float: one separately rounded multiply and add per k, ascending k from 0.0f, which
//     is the summation order of the reference CPU GEMM
//     (TileProgramming/tensor_utils.cu:34-45), so fp32 results equal it bit for bit;
//   - int8: exact int32.
#include "common.h"

namespace cig {
namespace {

constexpr int GT = 64;   // tile edge
constexpr int GK = 16;   // slab depth
constexpr int GPAD = 4;  // LDS row padding (floats / ints)

struct MacF32 {
  typedef float acc_t;
  static __device__ __forceinline__ float mac(float acc, float a, float b) {
    return __fadd_rn(acc, __fmul_rn(a, b));
  }
};
struct MacI32 {
  typedef int32_t acc_t;
  static __device__ __forceinline__ int32_t mac(int32_t acc, int32_t a, int32_t b) {
    return acc + a * b;
  }
};

struct LoadF32 {
  static __device__ __forceinline__ float get(const float* p) { return *p; }
};
template <typename E16>
struct Load16 {
  static __device__ __forceinline__ float get(const uint16_t* p) { return E16::widen(*p); }
};
struct LoadI8 {
  static __device__ __forceinline__ int32_t get(const int8_t* p) { return (int32_t)*p; }
};

template <typename TIn, typename Load, typename Mac, bool B_NK, typename Epi>
__global__ __launch_bounds__(256) void gemm_generic_kernel(int64_t M, int64_t N, int64_t K,
                                                           const TIn* __restrict__ A,
                                                           int64_t lda,
                                                           const TIn* __restrict__ B,
                                                           int64_t ldb, Epi epi) {
  typedef typename Mac::acc_t acc_t;
  __shared__ acc_t As[GK][GT + GPAD];  // [k][m]
  __shared__ acc_t Bs[GK][GT + GPAD];  // [k][n]

  const int t = threadIdx.x;
  const int tx = t % 16, ty = t / 16;
  const int64_t m0 = (int64_t)blockIdx.y * GT;
  const int64_t n0 = (int64_t)blockIdx.x * GT;

  acc_t acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0;

  for (int64_t k0 = 0; k0 < K; k0 += GK) {
    // A slab: 64 rows x 16 k = 1024 elements, 4 per thread, k fastest (contiguous in A).
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int e = t + i * 256;
      const int kk = e % GK, mm = e / GK;
      const int64_t gm = m0 + mm, gk = k0 + kk;
      As[kk][mm] = (gm < M && gk < K) ? Load::get(A + gm * lda + gk) : (acc_t)0;
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int e = t + i * 256;
      int kk, nn;
      if (B_NK) {  // B is N x K: k contiguous
        kk = e % GK;
        nn = e / GK;
      } else {  // B is K x N: n contiguous
        nn = e % GT;
        kk = e / GT;
      }
      const int64_t gn = n0 + nn, gk = k0 + kk;
      acc_t v = 0;
      if (gn < N && gk < K) v = Load::get(B_NK ? B + gn * ldb + gk : B + gk * ldb + gn);
      Bs[kk][nn] = v;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < GK; ++kk) {
      acc_t a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = As[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j] = Bs[kk][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = Mac::mac(acc[i][j], a[i], b[j]);
    }
    __syncthreads();
  }

#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int64_t gm = m0 + ty * 4 + i;
    if (gm >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int64_t gn = n0 + tx * 4 + j;
      if (gn < N) epi(gm, gn, acc[i][j]);
    }
  }
}

inline dim3 generic_grid(int64_t M, int64_t N) {
  return dim3((unsigned)((N + GT - 1) / GT), (unsigned)((M + GT - 1) / GT), 1);
}

}  // namespace

void launch_generic_f32(cigemmContext* ctx, int64_t M, int64_t N, int64_t K, const float* A,
                        int64_t lda, const float* B, int64_t ldb, float* C, int64_t ldc,
                        const BiasAct* ba) {
  if (ba) {
    EpiBiasActF32 epi{C, ldc, ba->bias, ba->relu};
    hipLaunchKernelGGL((gemm_generic_kernel<float, LoadF32, MacF32, false, EpiBiasActF32>),
                       generic_grid(M, N), dim3(256), 0, ctx->stream, M, N, K, A, lda, B, ldb, epi);
    ctx->last_kernel = "f32_generic_64x64x16_bias_act";
    return;
  }
  EpiStoreF32 epi{C, ldc};
  hipLaunchKernelGGL((gemm_generic_kernel<float, LoadF32, MacF32, false, EpiStoreF32>),
                     generic_grid(M, N), dim3(256), 0, ctx->stream, M, N, K, A, lda, B, ldb, epi);
  ctx->last_kernel = "f32_generic_64x64x16";
}

void launch_generic_16(cigemmContext* ctx, bool bf16, int64_t M, int64_t N, int64_t K,
                       const uint16_t* A, int64_t lda, const uint16_t* B, int64_t ldb,
                       uint16_t* C, int64_t ldc) {
  if (bf16) {
    EpiStore16<BF16> epi{C, ldc};
    hipLaunchKernelGGL(
        (gemm_generic_kernel<uint16_t, Load16<BF16>, MacF32, false, EpiStore16<BF16>>),
        generic_grid(M, N), dim3(256), 0, ctx->stream, M, N, K, A, lda, B, ldb, epi);
    ctx->last_kernel = "bf16_generic_64x64x16";
  } else {
    EpiStore16<F16> epi{C, ldc};
    hipLaunchKernelGGL(
        (gemm_generic_kernel<uint16_t, Load16<F16>, MacF32, false, EpiStore16<F16>>),
        generic_grid(M, N), dim3(256), 0, ctx->stream, M, N, K, A, lda, B, ldb, epi);
    ctx->last_kernel = "f16_generic_64x64x16";
  }
}

template <bool B_NK, typename Epi>
static void launch_i8_with(cigemmContext* ctx, int64_t M, int64_t N, int64_t K, const int8_t* A,
                           int64_t lda, const int8_t* B, int64_t ldb, const Epi& epi) {
  hipLaunchKernelGGL((gemm_generic_kernel<int8_t, LoadI8, MacI32, B_NK, Epi>), generic_grid(M, N),
                     dim3(256), 0, ctx->stream, M, N, K, A, lda, B, ldb, epi);
}

template <bool B_NK>
static void launch_i8_layout(cigemmContext* ctx, int64_t M, int64_t N, int64_t K,
                             const int8_t* A, int64_t lda, const int8_t* B, int64_t ldb,
                             int32_t* C, int64_t ldc, const DequantArgs* dq) {
  if (!dq) {
    launch_i8_with<B_NK>(ctx, M, N, K, A, lda, B, ldb, EpiStoreI32{C, ldc});
    return;
  }
  const bool dump = dq->acc_out != nullptr;
#define CIG_DQ(OB, DA)                                                                       \
  launch_i8_with<B_NK>(ctx, M, N, K, A, lda, B, ldb,                                         \
                       EpiDequant<OB, DA>{dq->out, dq->ldo, dq->sa, dq->sb, dq->sa_vec,      \
                                          dq->sb_vec, dq->acc_out, dq->ldacc})
  if (dq->out_bf16) {
    if (dump) CIG_DQ(true, true); else CIG_DQ(true, false);
  } else {
    if (dump) CIG_DQ(false, true); else CIG_DQ(false, false);
  }
#undef CIG_DQ
}

void launch_generic_i8(cigemmContext* ctx, int64_t M, int64_t N, int64_t K, const int8_t* A,
                       int64_t lda, const int8_t* B, int64_t ldb, bool b_nk, int32_t* C,
                       int64_t ldc, const DequantArgs* dq) {
  if (b_nk)
    launch_i8_layout<true>(ctx, M, N, K, A, lda, B, ldb, C, ldc, dq);
  else
    launch_i8_layout<false>(ctx, M, N, K, A, lda, B, ldb, C, ldc, dq);
  ctx->last_kernel = dq ? "i8_generic_64x64x16_dequant" : "i8_generic_64x64x16";
}

}  // namespace cig
