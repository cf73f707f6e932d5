// fp32 GEMM placeholder gate: no MFMA family yet, every shape goes to the any-shape kernel.
#include "common.h"
namespace cig {
bool launch_f32_mfma(cigemmContext*, int64_t, int64_t, int64_t, const float*, int64_t,
                     const float*, int64_t, float*, int64_t) { return false; }
}  // namespace cig
