// CPU test of the suite's host logic: the timing protocol with a fake clock
// (quantization/GEMM_bf16.cu:59-84) and the driver's two stdout formats
// (quantization/main.cu:13-19, 24-26).  Exits non-zero on the first failure.
#include <cmath>
#include <cstdio>
#include <sstream>
#include <string>

#include "gemm_timing.h"
#include "suite_format.h"

static int failures = 0;
#define EXPECT(cond)                                                       \
  do {                                                                     \
    if (!(cond)) {                                                         \
      std::printf("FAIL %s:%d: %s\n", __FILE__, __LINE__, #cond);          \
      ++failures;                                                          \
    }                                                                      \
  } while (0)

int main() {
  // Fake clock: every launch costs `per_iter` seconds of device time, visible to the host
  // only after a sync (the clock is read right after one).
  for (double per_iter : {1e-6, 3.7e-4, 2.5e-3, 0.05, 20.0}) {
    for (double budget : {0.0, 0.5, 10.0}) {
      double device_time = 0.0, host_time = 100.0;
      uint64_t launches = 0, syncs = 0;
      auto r = timed_gemm_loop(
          budget, [&] { device_time += per_iter; ++launches; },
          [&] { host_time = 100.0 + device_time; ++syncs; }, [&] { return host_time; });
      EXPECT(r.iters == launches);
      EXPECT(r.iters % 256 == 0);                       // clock only sampled every 256 launches
      EXPECT(r.secs >= budget);                         // never stops early
      EXPECT(std::fabs(r.secs - per_iter * r.iters) < 1e-9 * (1 + r.secs));
      if (budget > 0) {
        EXPECT(r.iters >= 256);
        // stops at the first sample at or past the budget: the previous sample was short of it
        EXPECT(per_iter * (r.iters - 256) < budget);
        EXPECT(syncs == r.iters / 256 + 1);             // one per sample + the final one
      } else {
        EXPECT(r.iters == 0);
      }
    }
  }
  // tflops = 2*M*N*K*iters / (secs * 1e12)
  EXPECT(gemm_tflops(4096, 4096, 4096, 256, 10.0) == 2.0 * 4096.0 * 4096.0 * 4096.0 * 256.0 / 1e13);
  EXPECT(std::fabs(gemm_tflops(8192, 8192, 8192, 1, 1e-3) - 1099.511627776) < 1e-9);

  // stdout formats
  std::ostringstream os;
  print_running(os, "BF16");
  EXPECT(os.str() == "Running BF16...\n");
  os.str("");
  GemmResult res{"INT8", 2816, 10.0123, 37.5};
  print_result(os, res);
  EXPECT(os.str() == "Ran 2816 INT8 GEMMs in 10.0123 s (37.5 TFLOP/s)\n");
  os.str("");
  GemmResult res2{"FP32", 256, 12.0, 0.123456789};
  print_result(os, res2);
  EXPECT(os.str() == "Ran 256 FP32 GEMMs in 12 s (0.123457 TFLOP/s)\n");   // default ostream precision 6

  // record layout (quantization/gemm_common.h:57-62)
  static_assert(sizeof(GemmResult) == 32, "GemmResult is {const char*, uint64_t, double, double}");
  static_assert(offsetof(GemmResult, iters) == 8 && offsetof(GemmResult, secs) == 16 &&
                    offsetof(GemmResult, tflops) == 24, "field order");

  if (failures) return 1;
  std::printf("host protocol OK\n");
  return 0;
}
