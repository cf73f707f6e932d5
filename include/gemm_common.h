/*
 * gemm_common.h -- drop-in counterpart of the reference suite's header of the same name
 * (quantization/gemm_common.h).  Same record, same four benchmark entry points; the
 * cuBLAS handle in their signature is replaced by this library's handle.
 *
 * A driver written against the reference header changes three things:
 *   cublasHandle_t          -> gemmHandle_t              (gemm_common.h:64-67)
 *   cublasCreate/Destroy    -> cigemmCreate/cigemmDestroy (main.cu:10,29)
 *   CHECK_CUDA/CHECK_CUBLAS -> CHECK_HIP/CHECK_GEMM       (gemm_common.h:37-55)
 */
#pragma once

#include <hip/hip_runtime_api.h>

#include <cstdint>
#include <cstdlib>
#include <iostream>

#include "cigemm.h"

typedef cigemmHandle_t gemmHandle_t;

/* quantization/gemm_common.h:10-35 */
inline const char* gemm_status_to_string(cigemmStatus_t status) {
  return cigemmGetStatusString(status);
}

/* quantization/gemm_common.h:37-45: print "<API> error: <text> at <file>:<line>", exit(1) */
#define CHECK_HIP(call)                                                       \
  do {                                                                        \
    hipError_t status_ = (call);                                              \
    if (status_ != hipSuccess) {                                              \
      std::cerr << "HIP error: " << hipGetErrorString(status_) << " at "      \
                << __FILE__ << ":" << __LINE__ << std::endl;                  \
      std::exit(EXIT_FAILURE);                                                \
    }                                                                         \
  } while (0)

/* quantization/gemm_common.h:47-55 */
#define CHECK_GEMM(call)                                                      \
  do {                                                                        \
    cigemmStatus_t status_ = (call);                                          \
    if (status_ != CIGEMM_STATUS_SUCCESS) {                                   \
      std::cerr << "cigemm error: " << gemm_status_to_string(status_)         \
                << " at " << __FILE__ << ":" << __LINE__ << std::endl;        \
      std::exit(EXIT_FAILURE);                                                \
    }                                                                         \
  } while (0)

/* quantization/gemm_common.h:57-62.  For INT8 the field named tflops holds TOPS
 * (quantization/GEMM_int8.cu:80-90). */
struct GemmResult {
  const char* name;
  uint64_t iters;
  double secs;
  double tflops;
};

/* quantization/gemm_common.h:64-67.  Each call allocates its operands, fills them on the
 * device with the reference generator, runs one warm-up GEMM, then back-to-back GEMMs
 * until the time budget is spent, and frees its buffers (quantization/GEMM_bf16.cu:21-91). */
GemmResult run_gemm_bf16(gemmHandle_t handle);
GemmResult run_gemm_fp16(gemmHandle_t handle);
GemmResult run_gemm_fp32(gemmHandle_t handle);
GemmResult run_gemm_int8(gemmHandle_t handle);

/* The reference hard-codes 4096^3 and a 10.0 s budget (GEMM_bf16.cu:22-24, 63).  These
 * setters exist so tests can run the same protocol quickly; the defaults are the
 * reference's values. */
void gemm_suite_set_seconds(double seconds);
void gemm_suite_set_size(int64_t m, int64_t n, int64_t k);
