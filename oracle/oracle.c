/*
 * CPU oracle for the quantization GEMM path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file restates, in plain C, the algorithms the reference repo uses on (or beside)
 * its quantization/ GEMM suite.  It is a checker: only tests/, the smoke check and the
 * cpu_baseline leg of bench.py may load it.  The shipped library never links it and has
 * no CPU fallback.
 *
 * Paths are relative to the reference repository root.
 *
 * Pinning status of each function (what, other than this file, fixes its answers):
 *   oracle_hash64 / oracle_fill_random_*   closed form of quantization/GEMM_*.cu fill
 *                                          kernels; pinned by hand-derived known answers
 *                                          (tests/golden/fill_random_kat.json).
 *   oracle_f32_to_bf16 / _f16 / widening   IEEE-754 RNE; pinned exhaustively against
 *                                          numpy float16 and a bit-level bf16 rule.
 *   oracle_matrixMulCPU, oracle_gemm_*     GEMM definition; pinned by identity / one-hot /
 *                                          exact-arithmetic inputs, integer closed forms,
 *                                          int64 and fp64 cross-checks, numpy.
 *   oracle_dequant_*                       build-defined epilogue (the reference stops at
 *                                          raw int32: quantization/GEMM_int8.cu:48-56);
 *                                          pinned against numpy float32 arithmetic.
 *   oracle_quantize_rows_i8                build-defined; pinned by hand cases.
 *   oracle_linear_f32                      MNIST MLP forward layer; pinned by bias-only,
 *                                          identity-weight and ReLU sign cases and numpy.
 *   cuBLAS's own summation order           parity unpinned: closed source, absent, and the
 *                                          reference holds no output for it.
 *
 * Compile with -ffp-contract=off so that no multiply-add is fused: the results are then
 * independent of compiler and host ISA.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

#define ORACLE_API __attribute__((visibility("default")))

ORACLE_API int oracle_num_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

/* ------------------------------------------------------------------------------------ */
/* Input generators: quantization/GEMM_fp32.cu:7-17, GEMM_bf16.cu:8-19,                 */
/* GEMM_fp16.cu:8-19, GEMM_int8.cu:8-19.                                                */
/* ------------------------------------------------------------------------------------ */

/* One LCG step of (idx ^ seed), modulo 2^64 (GEMM_fp32.cu:13-14). */
ORACLE_API uint64_t oracle_hash64(int64_t idx, uint64_t seed) {
  uint64_t x = (uint64_t)idx ^ seed;
  x = x * 2862933555777941757ULL + 3037000493ULL;
  return x;
}

/* 24-bit uniform in [0,1] then affine map (GEMM_fp32.cu:15-16). */
static inline float hash_to_float(uint64_t x, float lo, float hi) {
  float r = (float)((x >> 11) & 0xFFFFFF) / 16777215.0f;
  return lo + r * (hi - lo);
}

ORACLE_API void oracle_fill_random_f32(float* data, int64_t count, uint64_t seed, float lo,
                                       float hi) {
  for (int64_t idx = 0; idx < count; ++idx)
    data[idx] = hash_to_float(oracle_hash64(idx, seed), lo, hi);
}

/* ---- 16-bit narrowing: what __float2bfloat16 / __float2half do (round to nearest even),
 * GEMM_bf16.cu:18, GEMM_fp16.cu:18, TileProgramming/tensor_utils.h:65-72. ---- */

static inline uint32_t f32_bits(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  return u;
}
static inline float bits_f32(uint32_t u) {
  float f;
  memcpy(&f, &u, 4);
  return f;
}

ORACLE_API uint16_t oracle_f32_to_bf16(float f) {
  uint32_t u = f32_bits(f);
  if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((u >> 16) | 0x0040u); /* quiet NaN */
  uint32_t lsb = (u >> 16) & 1u;
  u += 0x7FFFu + lsb;
  return (uint16_t)(u >> 16);
}

ORACLE_API float oracle_bf16_to_f32(uint16_t h) { return bits_f32((uint32_t)h << 16); }

ORACLE_API uint16_t oracle_f32_to_f16(float f) {
  uint32_t u = f32_bits(f);
  uint32_t sign = (u >> 16) & 0x8000u;
  uint32_t absu = u & 0x7FFFFFFFu;
  if (absu > 0x7F800000u) return (uint16_t)(sign | 0x7E00u | ((absu >> 13) & 0x3FFu)); /* NaN */
  if (absu >= 0x47800000u) return (uint16_t)(sign | 0x7C00u); /* >= 65536 (or inf) -> inf   */
  if (absu < 0x33000000u) return (uint16_t)sign;              /* < 2^-25 -> +-0            */
  int32_t exp = (int32_t)(absu >> 23) - 127;                  /* unbiased                  */
  uint32_t man = (absu & 0x7FFFFFu) | 0x800000u;              /* 24-bit significand        */
  uint32_t shift;                                             /* bits dropped from `man`   */
  uint32_t base;                                              /* half bits before mantissa */
  if (exp >= -14) {                                           /* normal half               */
    shift = 13;
    base = (uint32_t)(exp + 15) << 10;
    man &= 0x7FFFFFu;
  } else {                                                    /* subnormal half            */
    shift = (uint32_t)(13 + (-14 - exp));
    base = 0;
  }
  uint32_t kept = man >> shift;
  uint32_t rem = man & ((1u << shift) - 1u);
  uint32_t half = 1u << (shift - 1);
  uint32_t out = base + kept;
  if (rem > half || (rem == half && (kept & 1u))) out += 1u; /* carry may reach exponent/inf */
  return (uint16_t)(sign | out);
}

ORACLE_API float oracle_f16_to_f32(uint16_t h) {
  uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1Fu;
  uint32_t man = h & 0x3FFu;
  if (exp == 0x1Fu) return bits_f32(sign | 0x7F800000u | (man << 13));
  if (exp == 0) {
    if (man == 0) return bits_f32(sign);
    /* subnormal: value = man * 2^-24, exact in float */
    float v = (float)man * 5.9604644775390625e-08f;
    return sign ? -v : v;
  }
  return bits_f32(sign | ((exp + 112u) << 23) | (man << 13));
}

ORACLE_API void oracle_f32_to_bf16_n(const float* in, uint16_t* out, int64_t n) {
  for (int64_t i = 0; i < n; ++i) out[i] = oracle_f32_to_bf16(in[i]);
}
ORACLE_API void oracle_f32_to_f16_n(const float* in, uint16_t* out, int64_t n) {
  for (int64_t i = 0; i < n; ++i) out[i] = oracle_f32_to_f16(in[i]);
}
ORACLE_API void oracle_bf16_to_f32_n(const uint16_t* in, float* out, int64_t n) {
  for (int64_t i = 0; i < n; ++i) out[i] = oracle_bf16_to_f32(in[i]);
}
ORACLE_API void oracle_f16_to_f32_n(const uint16_t* in, float* out, int64_t n) {
  for (int64_t i = 0; i < n; ++i) out[i] = oracle_f16_to_f32(in[i]);
}

ORACLE_API void oracle_fill_random_bf16(uint16_t* data, int64_t count, uint64_t seed, float lo,
                                        float hi) {
  for (int64_t idx = 0; idx < count; ++idx)
    data[idx] = oracle_f32_to_bf16(hash_to_float(oracle_hash64(idx, seed), lo, hi));
}

ORACLE_API void oracle_fill_random_f16(uint16_t* data, int64_t count, uint64_t seed, float lo,
                                       float hi) {
  for (int64_t idx = 0; idx < count; ++idx)
    data[idx] = oracle_f32_to_f16(hash_to_float(oracle_hash64(idx, seed), lo, hi));
}

/* 16-bit field of the hash, modulo the range width (GEMM_int8.cu:14-18). */
ORACLE_API void oracle_fill_random_i8(int8_t* data, int64_t count, uint64_t seed, int lo, int hi) {
  for (int64_t idx = 0; idx < count; ++idx) {
    uint64_t x = oracle_hash64(idx, seed);
    int r = (int)((x >> 11) & 0xFFFF);
    int val = lo + (r % (hi - lo + 1));
    data[idx] = (int8_t)val;
  }
}

/* ------------------------------------------------------------------------------------ */
/* GEMM: TileProgramming/tensor_utils.cu:34-45.                                          */
/* ------------------------------------------------------------------------------------ */

/* The reference function itself: square, row-major, i-j-k, float accumulator from 0. */
ORACLE_API void oracle_matrixMulCPU(float* C, const float* A, const float* B, int width) {
  for (int i = 0; i < width; ++i) {
    for (int j = 0; j < width; ++j) {
      float sum = 0.0f;
      for (int k = 0; k < width; ++k) {
        sum += A[i * width + k] * B[k * width + j];
      }
      C[i * width + j] = sum;
    }
  }
}

/* Same loop, rectangular with leading dimensions, rows [row0,row1) only.  Literal i-j-k
 * order; this is the form timed as the CPU baseline. */
ORACLE_API void oracle_gemm_f32_ijk(int64_t M, int64_t N, int64_t K, const float* A, int64_t lda,
                                    const float* B, int64_t ldb, float* C, int64_t ldc,
                                    int64_t row0, int64_t row1) {
  (void)M;
#pragma omp parallel for schedule(static)
  for (int64_t i = row0; i < row1; ++i) {
    for (int64_t j = 0; j < N; ++j) {
      float sum = 0.0f;
      for (int64_t k = 0; k < K; ++k) {
        sum += A[i * lda + k] * B[k * ldb + j];
      }
      C[i * ldc + j] = sum;
    }
  }
}

/* Every element still accumulates its products one at a time in ascending k, starting
 * from 0.0f, with separate multiply and add, so each C[i][j] is bit-identical to the
 * i-j-k loop above; only the interleaving across different j changes (cache friendly,
 * vectorisable over j).  tests/ prove the identity on random inputs. */
ORACLE_API void oracle_gemm_f32(int64_t M, int64_t N, int64_t K, const float* A, int64_t lda,
                                const float* B, int64_t ldb, float* C, int64_t ldc) {
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < M; ++i) {
    float* c = C + i * ldc;
    for (int64_t j = 0; j < N; ++j) c[j] = 0.0f;
    for (int64_t k = 0; k < K; ++k) {
      const float a = A[i * lda + k];
      const float* b = B + k * ldb;
      for (int64_t j = 0; j < N; ++j) c[j] += a * b[j];
    }
  }
}

/* fp64 checker for the fp32/fp16/bf16 kernels: inputs are the (already rounded) values
 * widened to float; products and sums in double.  Optionally also S = sum |a||b|, the
 * scale of the K-dependent error bound.  Rows [row0,row1), written at C[(i-row0)*ldc]. */
ORACLE_API void oracle_gemm_f64_rows(int64_t N, int64_t K, const float* A, int64_t lda,
                                     const float* B, int64_t ldb, double* C, double* S,
                                     int64_t ldc, int64_t row0, int64_t row1) {
#pragma omp parallel for schedule(static)
  for (int64_t i = row0; i < row1; ++i) {
    double* c = C + (i - row0) * ldc;
    double* s = S ? S + (i - row0) * ldc : NULL;
    for (int64_t j = 0; j < N; ++j) c[j] = 0.0;
    if (s)
      for (int64_t j = 0; j < N; ++j) s[j] = 0.0;
    for (int64_t k = 0; k < K; ++k) {
      const double a = (double)A[i * lda + k];
      const float* b = B + k * ldb;
      for (int64_t j = 0; j < N; ++j) c[j] += a * (double)b[j];
      if (s) {
        const double aa = fabs(a);
        for (int64_t j = 0; j < N; ++j) s[j] += aa * fabs((double)b[j]);
      }
    }
  }
}

/* int8 x int8 -> int32 twin of matrixMulCPU.  Integer sums are order independent, so the
 * cache-friendly loop order gives exactly the i-j-k result.  b_is_nk = 0: B is K x N
 * (row-major, like A.B in the reference); 1: B is N x K (each output channel's weights
 * contiguous), C = A . B^T. */
ORACLE_API void oracle_gemm_i8_i32(int64_t M, int64_t N, int64_t K, const int8_t* A, int64_t lda,
                                   const int8_t* B, int64_t ldb, int b_is_nk, int32_t* C,
                                   int64_t ldc) {
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < M; ++i) {
    int32_t* c = C + i * ldc;
    if (!b_is_nk) {
      for (int64_t j = 0; j < N; ++j) c[j] = 0;
      for (int64_t k = 0; k < K; ++k) {
        const int32_t a = A[i * lda + k];
        const int8_t* b = B + k * ldb;
        for (int64_t j = 0; j < N; ++j) c[j] += a * (int32_t)b[j];
      }
    } else {
      const int8_t* a = A + i * lda;
      for (int64_t j = 0; j < N; ++j) {
        const int8_t* b = B + j * ldb;
        int32_t sum = 0;
        for (int64_t k = 0; k < K; ++k) sum += (int32_t)a[k] * (int32_t)b[k];
        c[j] = sum;
      }
    }
  }
}

/* Literal i-j-k int8 loop with a 64-bit accumulator: cross-check for the above. */
ORACLE_API void oracle_gemm_i8_i64_ijk(int64_t M, int64_t N, int64_t K, const int8_t* A,
                                       int64_t lda, const int8_t* B, int64_t ldb, int b_is_nk,
                                       int64_t* C, int64_t ldc) {
  for (int64_t i = 0; i < M; ++i)
    for (int64_t j = 0; j < N; ++j) {
      int64_t sum = 0;
      for (int64_t k = 0; k < K; ++k) {
        int64_t b = b_is_nk ? B[j * ldb + k] : B[k * ldb + j];
        sum += (int64_t)A[i * lda + k] * b;
      }
      C[i * ldc + j] = sum;
    }
}

/* ------------------------------------------------------------------------------------ */
/* Dequantize epilogue (build-defined): out = ((float)acc * sA_i) * sB_j, left to right, */
/* each operation rounded to fp32, no fusion.  sa_per_row / sb_per_col = 0: one scale.   */
/* ------------------------------------------------------------------------------------ */
ORACLE_API void oracle_dequant_f32(int64_t M, int64_t N, const int32_t* acc, int64_t ldacc,
                                   const float* sa, int sa_per_row, const float* sb,
                                   int sb_per_col, float* out, int64_t ldo) {
  for (int64_t i = 0; i < M; ++i) {
    const float a = sa[sa_per_row ? i : 0];
    for (int64_t j = 0; j < N; ++j) {
      const float b = sb[sb_per_col ? j : 0];
      float t = (float)acc[i * ldacc + j] * a;
      out[i * ldo + j] = t * b;
    }
  }
}

ORACLE_API void oracle_dequant_bf16(int64_t M, int64_t N, const int32_t* acc, int64_t ldacc,
                                    const float* sa, int sa_per_row, const float* sb,
                                    int sb_per_col, uint16_t* out, int64_t ldo) {
  for (int64_t i = 0; i < M; ++i) {
    const float a = sa[sa_per_row ? i : 0];
    for (int64_t j = 0; j < N; ++j) {
      const float b = sb[sb_per_col ? j : 0];
      float t = (float)acc[i * ldacc + j] * a;
      out[i * ldo + j] = oracle_f32_to_bf16(t * b);
    }
  }
}

/* Symmetric absmax quantizer along the contiguous axis (build-defined):
 * s = absmax/127 (1 if the row is all zero), q = clamp(nearbyint(x / s), -127, 127),
 * ties to even. */
ORACLE_API void oracle_quantize_rows_i8(int64_t rows, int64_t cols, const float* x, int64_t ldx,
                                        int8_t* q, int64_t ldq, float* scale) {
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < rows; ++i) {
    float amax = 0.0f;
    for (int64_t j = 0; j < cols; ++j) {
      float v = fabsf(x[i * ldx + j]);
      if (v > amax) amax = v;
    }
    float s = amax > 0.0f ? amax / 127.0f : 1.0f;
    scale[i] = s;
    for (int64_t j = 0; j < cols; ++j) {
      float r = nearbyintf(x[i * ldx + j] / s);
      if (r > 127.0f) r = 127.0f;
      if (r < -127.0f) r = -127.0f;
      q[i * ldq + j] = (int8_t)r;
    }
  }
}

/* ------------------------------------------------------------------------------------ */
/* MLP forward layer of the MNIST demo: MNIST/mnist_nn.cu:10-24 (input -> hidden),       */
/* 27-33 (ReLU), 36-49 (hidden -> output).  sum starts at the bias and adds the products */
/* one at a time in ascending i; W is input-major (W[i * N + j]).                        */
/* ------------------------------------------------------------------------------------ */
ORACLE_API void oracle_linear_f32(int64_t M, int64_t N, int64_t K, const float* X, const float* W,
                                  const float* bias, int relu, float* out) {
#pragma omp parallel for schedule(static)
  for (int64_t b = 0; b < M; ++b) {
    float* o = out + b * N;
    for (int64_t j = 0; j < N; ++j) o[j] = bias ? bias[j] : 0.0f;
    for (int64_t i = 0; i < K; ++i) {
      const float x = X[b * K + i];
      const float* w = W + i * N;
      for (int64_t j = 0; j < N; ++j) o[j] += x * w[j];
    }
    if (relu)
      for (int64_t j = 0; j < N; ++j) o[j] = fmaxf(0.0f, o[j]);
  }
}

/* ------------------------------------------------------------------------------------ */
/* Compare: TileProgramming/matmulTensor.cu:18-28 (absolute eps, first mismatch wins).   */
/* Returns -1 when all width*width entries agree, else the index of the first mismatch.  */
/* ------------------------------------------------------------------------------------ */
ORACLE_API int64_t oracle_checkResult(const float* GPU, const float* CPU, int width, float eps,
                                      int verbose) {
  int64_t size = (int64_t)width * width;
  for (int64_t i = 0; i < size; ++i) {
    if (fabs((double)GPU[i] - (double)CPU[i]) > (double)eps) {
      if (verbose) printf("Mismatch at %lld: GPU=%f, CPU=%f\n", (long long)i, GPU[i], CPU[i]);
      return i;
    }
  }
  return -1;
}
