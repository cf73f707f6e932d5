// Skinny (decode-shape) GEMM placeholder gate.
#include "common.h"
namespace cig {
bool launch_skinny_16(cigemmContext*, bool, int64_t, int64_t, int64_t, const uint16_t*, int64_t,
                      const uint16_t*, int64_t, uint16_t*, int64_t) { return false; }
bool launch_skinny_i8(cigemmContext*, int64_t, int64_t, int64_t, const int8_t*, int64_t,
                      const int8_t*, int64_t, bool, int32_t*, int64_t, const DequantArgs*) { return false; }
}  // namespace cig
