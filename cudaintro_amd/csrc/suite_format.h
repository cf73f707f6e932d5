// The two stdout formats of the reference driver (quantization/main.cu:13-19, 24-26).
#pragma once

#include <ostream>

#include "gemm_common.h"

inline void print_running(std::ostream& os, const char* name) {
  os << "Running " << name << "..." << std::endl;
}

inline void print_result(std::ostream& os, const GemmResult& result) {
  os << "Ran " << result.iters << " " << result.name << " GEMMs in " << result.secs << " s ("
     << result.tflops << " TFLOP/s)\n";
}
