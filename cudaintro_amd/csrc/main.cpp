// gemm_suite: the reference driver's flow (quantization/main.cu:8-31) -- create the handle,
// run BF16, FP16, FP32, INT8 in that order, print one line per result, destroy the handle.
// With no arguments it is the reference run (4096^3, 10 s per precision).
//   --seconds S      time budget per precision (default 10)
//   --size N         M = N = K (default 4096)
#include <cstdlib>
#include <cstring>
#include <iostream>

#include "gemm_common.h"
#include "suite_format.h"

int main(int argc, char** argv) {
  for (int i = 1; i < argc; ++i) {
    if (!std::strcmp(argv[i], "--seconds") && i + 1 < argc) {
      gemm_suite_set_seconds(std::atof(argv[++i]));
    } else if (!std::strcmp(argv[i], "--size") && i + 1 < argc) {
      const long long n = std::atoll(argv[++i]);
      gemm_suite_set_size(n, n, n);
    } else {
      std::cerr << "usage: gemm_suite [--seconds S] [--size N]" << std::endl;
      return 2;
    }
  }

  gemmHandle_t handle = nullptr;
  CHECK_GEMM(cigemmCreate(&handle));

  print_running(std::cout, "BF16");
  GemmResult bf16 = run_gemm_bf16(handle);
  print_running(std::cout, "FP16");
  GemmResult fp16 = run_gemm_fp16(handle);
  print_running(std::cout, "FP32");
  GemmResult fp32 = run_gemm_fp32(handle);
  print_running(std::cout, "INT8");
  GemmResult int8 = run_gemm_int8(handle);

  const GemmResult results[] = {bf16, fp16, fp32, int8};
  for (const auto& result : results) print_result(std::cout, result);

  CHECK_GEMM(cigemmDestroy(handle));
  return 0;
}
