/* Exercises every function of oracle/oracle.c on small exactly sized heap buffers (ragged
 * shapes, leading dimensions larger than the rows, empty inputs), for a build with
 * -fsanitize=address,undefined: any read or write past a buffer, signed overflow, misaligned
 * access or invalid conversion aborts the program.  It also cross-checks a few results, so
 * that the sanitized build is known to compute the same thing. */
#include "../../oracle/oracle.c"

#include <stdlib.h>

static unsigned long long lcg = 88172645463325252ull;
static int rnd(int lo, int hi) {
  lcg = lcg * 6364136223846793005ull + 1442695040888963407ull;
  return lo + (int)((lcg >> 33) % (unsigned long long)(hi - lo + 1));
}
#define CHECK(c) do { if (!(c)) { printf("FAILED %s:%d: %s\n", __FILE__, __LINE__, #c); return 1; } } while (0)

int main(void) {
  CHECK(oracle_num_threads() >= 1);
  static const int shapes[][3] = {{1, 1, 1}, {3, 5, 7}, {17, 33, 9}, {32, 32, 64}, {5, 1, 40}, {2, 129, 3}};
  for (unsigned s = 0; s < sizeof(shapes) / sizeof(shapes[0]); ++s) {
    const int M = shapes[s][0], N = shapes[s][1], K = shapes[s][2];
    const int lda = K + 3, ldb = N + 2, ldc = N + 1, ldbt = K + 1;
    /* exactly sized: the last row has no padding behind it */
    float* A = malloc(sizeof(float) * ((size_t)(M - 1) * lda + K));
    float* B = malloc(sizeof(float) * ((size_t)(K - 1) * ldb + N));
    float* C = malloc(sizeof(float) * ((size_t)(M - 1) * ldc + N));
    float* C2 = malloc(sizeof(float) * ((size_t)(M - 1) * ldc + N));
    double* D = malloc(sizeof(double) * ((size_t)(M - 1) * ldc + N));
    double* S = malloc(sizeof(double) * ((size_t)(M - 1) * ldc + N));
    int8_t* A8 = malloc((size_t)(M - 1) * lda + K);
    int8_t* B8 = malloc((size_t)(K - 1) * ldb + N);
    int8_t* B8t = malloc((size_t)(N - 1) * ldbt + K);
    int32_t* C32 = malloc(sizeof(int32_t) * ((size_t)(M - 1) * ldc + N));
    int32_t* C32t = malloc(sizeof(int32_t) * ((size_t)(M - 1) * ldc + N));
    int64_t* C64 = malloc(sizeof(int64_t) * ((size_t)(M - 1) * ldc + N));
    for (int i = 0; i < M; ++i)
      for (int k = 0; k < K; ++k) {
        A[i * lda + k] = (float)rnd(-8, 8) * 0.25f;
        A8[i * lda + k] = (int8_t)rnd(-127, 127);
      }
    for (int k = 0; k < K; ++k)
      for (int j = 0; j < N; ++j) {
        B[k * ldb + j] = (float)rnd(-8, 8) * 0.5f;
        B8[k * ldb + j] = (int8_t)rnd(-127, 127);
        B8t[j * ldbt + k] = B8[k * ldb + j];
      }
    oracle_gemm_f32(M, N, K, A, lda, B, ldb, C, ldc);
    oracle_gemm_f32_ijk(M, N, K, A, lda, B, ldb, C2, ldc, 0, M);
    oracle_gemm_f64_rows(N, K, A, lda, B, ldb, D, S, ldc, 0, M);
    oracle_gemm_f64_rows(N, K, A, lda, B, ldb, D, NULL, ldc, 0, M);
    for (int i = 0; i < M; ++i)
      for (int j = 0; j < N; ++j) {
        CHECK(C[i * ldc + j] == C2[i * ldc + j]);
        CHECK((double)C[i * ldc + j] == D[i * ldc + j]); /* exact inputs: every order agrees */
        CHECK(S[i * ldc + j] >= fabs(D[i * ldc + j]));
      }
    oracle_gemm_i8_i32(M, N, K, A8, lda, B8, ldb, 0, C32, ldc);
    oracle_gemm_i8_i32(M, N, K, A8, lda, B8t, ldbt, 1, C32t, ldc);
    oracle_gemm_i8_i64_ijk(M, N, K, A8, lda, B8, ldb, 0, C64, ldc);
    for (int i = 0; i < M; ++i)
      for (int j = 0; j < N; ++j) {
        CHECK(C32[i * ldc + j] == C32t[i * ldc + j]);
        CHECK((int64_t)C32[i * ldc + j] == C64[i * ldc + j]);
      }
    oracle_gemm_i8_i64_ijk(M, N, K, A8, lda, B8t, ldbt, 1, C64, ldc);
    for (int i = 0; i < M; ++i)
      for (int j = 0; j < N; ++j) CHECK((int64_t)C32[i * ldc + j] == C64[i * ldc + j]);
    /* dequant, both scale modes and output types */
    float* sa = malloc(sizeof(float) * M);
    float* sb = malloc(sizeof(float) * N);
    float* of = malloc(sizeof(float) * ((size_t)(M - 1) * ldc + N));
    uint16_t* ob = malloc(sizeof(uint16_t) * ((size_t)(M - 1) * ldc + N));
    for (int i = 0; i < M; ++i) sa[i] = 0.001f * (float)(i + 1);
    for (int j = 0; j < N; ++j) sb[j] = 0.002f * (float)(j + 1);
    for (int pr = 0; pr < 2; ++pr)
      for (int pc = 0; pc < 2; ++pc) {
        oracle_dequant_f32(M, N, C32, ldc, sa, pr, sb, pc, of, ldc);
        oracle_dequant_bf16(M, N, C32, ldc, sa, pr, sb, pc, ob, ldc);
        for (int i = 0; i < M; ++i)
          for (int j = 0; j < N; ++j) CHECK(ob[i * ldc + j] == oracle_f32_to_bf16(of[i * ldc + j]));
      }
    /* quantizer: a zero row, a spike, ordinary rows */
    int8_t* q = malloc((size_t)(M - 1) * lda + K);
    float* sc = malloc(sizeof(float) * M);
    for (int k = 0; k < K; ++k) A[k] = 0.0f;
    oracle_quantize_rows_i8(M, K, A, lda, q, lda, sc);
    CHECK(sc[0] == 1.0f);
    for (int k = 0; k < K; ++k) CHECK(q[k] == 0);
    for (int i = 1; i < M; ++i)
      for (int k = 0; k < K; ++k) CHECK(q[i * lda + k] >= -127 && q[i * lda + k] <= 127);
    /* linear layer (contiguous operands), with and without bias */
    float* X = malloc(sizeof(float) * (size_t)M * K);
    float* W = malloc(sizeof(float) * (size_t)K * N);
    float* o1 = malloc(sizeof(float) * (size_t)M * N);
    for (int i = 0; i < M * K; ++i) X[i] = (float)rnd(-4, 4) * 0.5f;
    for (int i = 0; i < K * N; ++i) W[i] = (float)rnd(-4, 4) * 0.25f;
    oracle_linear_f32(M, N, K, X, W, sb, 1, o1);
    for (int i = 0; i < M * N; ++i) CHECK(o1[i] >= 0.0f);
    oracle_linear_f32(M, N, K, X, W, NULL, 0, o1);
    free(A); free(B); free(C); free(C2); free(D); free(S); free(A8); free(B8); free(B8t); free(C32);
    free(C32t); free(C64); free(sa); free(sb); free(of); free(ob); free(q); free(sc); free(X); free(W);
    free(o1);
  }
  /* square forms and the compare */
  {
    const int w = 19;
    float* A = malloc(sizeof(float) * w * w);
    float* B = malloc(sizeof(float) * w * w);
    float* C = malloc(sizeof(float) * w * w);
    float* C2 = malloc(sizeof(float) * w * w);
    for (int i = 0; i < w * w; ++i) {
      A[i] = (float)rnd(-8, 8) * 0.125f;
      B[i] = (float)rnd(-8, 8) * 0.125f;
    }
    oracle_matrixMulCPU(C, A, B, w);
    oracle_gemm_f32(w, w, w, A, w, B, w, C2, w);
    CHECK(oracle_checkResult(C, C2, w, 0.0f, 0) == -1);
    C2[w * w - 1] += 1.0f;
    CHECK(oracle_checkResult(C, C2, w, 1e-5f, 0) == (int64_t)w * w - 1);
    free(A); free(B); free(C); free(C2);
  }
  /* generators: odd counts, zero count, known first values of the int8 stream */
  {
    const int64_t n = 1001;
    float* f = malloc(sizeof(float) * n);
    uint16_t* h = malloc(sizeof(uint16_t) * n);
    int8_t* b = malloc(n);
    oracle_fill_random_f32(f, n, 0x3234, -1.0f, 1.0f);
    oracle_fill_random_bf16(h, n, 0x1234, -1.0f, 1.0f);
    oracle_fill_random_f16(h, n, 0x2234, -1.0f, 1.0f);
    oracle_fill_random_i8(b, n, 0x4234, -127, 127);
    CHECK(b[0] == 22 && b[1] == 34 && b[2] == 46 && b[3] == 58 && b[4] == -27);
    CHECK(oracle_hash64(0, 0x1234) == 0x3b51bc5eb15ab091ull);
    for (int64_t i = 0; i < n; ++i) CHECK(f[i] >= -1.0f && f[i] <= 1.0f && b[i] >= -127);
    oracle_fill_random_f32(f, 0, 1, 0.0f, 1.0f);
    oracle_fill_random_i8(b, 0, 1, -1, 1);
    free(f); free(h); free(b);
  }
  /* conversions: every 16-bit pattern both ways, and awkward floats */
  {
    uint16_t* h = malloc(sizeof(uint16_t) * 65536);
    float* f = malloc(sizeof(float) * 65536);
    uint16_t* h2 = malloc(sizeof(uint16_t) * 65536);
    for (int i = 0; i < 65536; ++i) h[i] = (uint16_t)i;
    oracle_bf16_to_f32_n(h, f, 65536);
    oracle_f32_to_bf16_n(f, h2, 65536);
    for (int i = 0; i < 65536; ++i) CHECK(f[i] != f[i] || h2[i] == h[i]);
    oracle_f16_to_f32_n(h, f, 65536);
    oracle_f32_to_f16_n(f, h2, 65536);
    for (int i = 0; i < 65536; ++i) CHECK(f[i] != f[i] || h2[i] == h[i]);
    static const float awkward[] = {0.0f, -0.0f, 1e-45f, 1e-40f, 6e-8f, 6.1e-5f, 65504.0f, 65520.0f,
                                    1e10f, -1e10f, 3.4e38f, INFINITY, -INFINITY, NAN};
    for (unsigned i = 0; i < sizeof(awkward) / sizeof(awkward[0]); ++i) {
      (void)oracle_f32_to_f16(awkward[i]);
      (void)oracle_f32_to_bf16(awkward[i]);
    }
    free(h); free(f); free(h2);
  }
  printf("oracle sanitized OK\n");
  return 0;
}
