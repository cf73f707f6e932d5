// The reference suite's timing protocol (quantization/GEMM_bf16.cu:59-84), as a template
// over the clock so it can be tested on the CPU with a fake clock.
//
//   start = now(); iters = 0
//   while (now_sample - start < budget) { launch(); ++iters;
//        if ((iters & 0xFF) == 0) { sync(); now_sample = now(); } }
//   sync(); secs = now() - start
//   tflops = 2*M*N*K*iters / (secs * 1e12)
//
// Consequences the tests pin: iters is a multiple of 256, and secs >= budget.
#pragma once

#include <cstdint>

struct TimedLoopResult {
  uint64_t iters;
  double secs;
};

// Launch: void();  Sync: void();  Now: double() in seconds.
template <typename Launch, typename Sync, typename Now>
TimedLoopResult timed_gemm_loop(double budget_secs, Launch&& launch, Sync&& sync, Now&& now) {
  const double start = now();
  double sample = start;
  uint64_t iters = 0;
  while (sample - start < budget_secs) {
    launch();
    ++iters;
    if ((iters & 0xFF) == 0) {
      sync();
      sample = now();
    }
  }
  sync();
  const double end = now();
  return {iters, end - start};
}

inline double gemm_tflops(int64_t m, int64_t n, int64_t k, uint64_t iters, double secs) {
  const double flops_per_iter =
      2.0 * static_cast<double>(m) * static_cast<double>(n) * static_cast<double>(k);
  return (flops_per_iter * static_cast<double>(iters)) / (secs * 1.0e12);
}
