// The four benchmark entry points of the reference suite (quantization/GEMM_bf16.cu:21-91,
// GEMM_fp16.cu:21-91, GEMM_fp32.cu:19-89, GEMM_int8.cu:21-91) on top of the C ABI:
// allocate, fill on the device with the reference generator and seeds, one warm-up GEMM,
// the timed loop, free, return {name, iters, secs, tflops}.
#include <chrono>

#include "gemm_common.h"
#include "gemm_timing.h"

namespace {

double g_seconds = 10.0;                      // GEMM_bf16.cu:63
int64_t g_m = 4096, g_n = 4096, g_k = 4096;   // GEMM_bf16.cu:22-24

double steady_now() {
  return std::chrono::duration<double>(std::chrono::steady_clock::now().time_since_epoch())
      .count();
}

void* stream_of(gemmHandle_t handle) {
  void* s = nullptr;
  CHECK_GEMM(cigemmGetStream(handle, &s));
  return s;
}

// Allocate -> fill -> warm-up -> timed loop -> free, shared by the four precisions.
template <typename TIn, typename TOut, typename Fill, typename Gemm>
GemmResult run_one(gemmHandle_t handle, const char* name, Fill&& fill, Gemm&& gemm) {
  const int64_t M = g_m, N = g_n, K = g_k;
  TIn* a = nullptr;
  TIn* b = nullptr;
  TOut* c = nullptr;
  CHECK_HIP(hipMalloc(reinterpret_cast<void**>(&a), M * K * sizeof(TIn)));
  CHECK_HIP(hipMalloc(reinterpret_cast<void**>(&b), K * N * sizeof(TIn)));
  CHECK_HIP(hipMalloc(reinterpret_cast<void**>(&c), M * N * sizeof(TOut)));
  fill(a, M * K, b, K * N);
  CHECK_HIP(hipGetLastError());

  hipStream_t stream = static_cast<hipStream_t>(stream_of(handle));
  CHECK_GEMM(gemm(a, b, c));                       // warm-up
  CHECK_HIP(hipStreamSynchronize(stream));

  TimedLoopResult r = timed_gemm_loop(
      g_seconds, [&] { CHECK_GEMM(gemm(a, b, c)); },
      [&] { CHECK_HIP(hipStreamSynchronize(stream)); }, steady_now);

  const double tflops = gemm_tflops(M, N, K, r.iters, r.secs);
  CHECK_HIP(hipFree(c));
  CHECK_HIP(hipFree(a));
  CHECK_HIP(hipFree(b));
  return {name, r.iters, r.secs, tflops};
}

}  // namespace

void gemm_suite_set_seconds(double seconds) { g_seconds = seconds; }
void gemm_suite_set_size(int64_t m, int64_t n, int64_t k) {
  g_m = m;
  g_n = n;
  g_k = k;
}

GemmResult run_gemm_bf16(gemmHandle_t handle) {
  const int64_t M = g_m, N = g_n, K = g_k;
  return run_one<uint16_t, uint16_t>(
      handle, "BF16",
      [&](uint16_t* a, int64_t na, uint16_t* b, int64_t nb) {
        CHECK_GEMM(cigemm_fill_random_bf16(handle, a, na, 0x1234U, -1.0f, 1.0f));  // GEMM_bf16.cu:44
        CHECK_GEMM(cigemm_fill_random_bf16(handle, b, nb, 0x9876U, -1.0f, 1.0f));  // :45
      },
      [&](const uint16_t* a, const uint16_t* b, uint16_t* c) {
        return cigemm_gemm_bf16(handle, M, N, K, a, K, b, N, c, N);
      });
}

GemmResult run_gemm_fp16(gemmHandle_t handle) {
  const int64_t M = g_m, N = g_n, K = g_k;
  return run_one<uint16_t, uint16_t>(
      handle, "FP16",
      [&](uint16_t* a, int64_t na, uint16_t* b, int64_t nb) {
        CHECK_GEMM(cigemm_fill_random_f16(handle, a, na, 0x2234U, -1.0f, 1.0f));  // GEMM_fp16.cu:44
        CHECK_GEMM(cigemm_fill_random_f16(handle, b, nb, 0x8876U, -1.0f, 1.0f));  // :45
      },
      [&](const uint16_t* a, const uint16_t* b, uint16_t* c) {
        return cigemm_gemm_f16(handle, M, N, K, a, K, b, N, c, N);
      });
}

GemmResult run_gemm_fp32(gemmHandle_t handle) {
  const int64_t M = g_m, N = g_n, K = g_k;
  return run_one<float, float>(
      handle, "FP32",
      [&](float* a, int64_t na, float* b, int64_t nb) {
        CHECK_GEMM(cigemm_fill_random_f32(handle, a, na, 0x3234U, -1.0f, 1.0f));  // GEMM_fp32.cu:42
        CHECK_GEMM(cigemm_fill_random_f32(handle, b, nb, 0x7776U, -1.0f, 1.0f));  // :43
      },
      [&](const float* a, const float* b, float* c) {
        return cigemm_gemm_f32(handle, M, N, K, a, K, b, N, c, N);
      });
}

GemmResult run_gemm_int8(gemmHandle_t handle) {
  const int64_t M = g_m, N = g_n, K = g_k;
  return run_one<int8_t, int32_t>(
      handle, "INT8",
      [&](int8_t* a, int64_t na, int8_t* b, int64_t nb) {
        CHECK_GEMM(cigemm_fill_random_i8(handle, a, na, 0x4234U, -127, 127));  // GEMM_int8.cu:44
        CHECK_GEMM(cigemm_fill_random_i8(handle, b, nb, 0x6676U, -127, 127));  // :45
      },
      [&](const int8_t* a, const int8_t* b, int32_t* c) {
        return cigemm_gemm_i8_i32(handle, M, N, K, a, K, b, N, CIGEMM_B_KN, c, N);
      });
}
