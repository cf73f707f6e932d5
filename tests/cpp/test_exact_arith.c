/* Exhaustive host-side check of the two division-free forms the device fill kernels use
 * (cudaintro_amd/csrc/fill_quant.hip): they must equal the plain C expressions of the
 * reference generators (quantization/GEMM_fp32.cu:13-15, GEMM_int8.cu:14-17) for every
 * possible operand.  fmaf here and the device's fused multiply-add are the same IEEE
 * operation; the file is built with -ffp-contract=off. */
#include <math.h>
#include <stdint.h>
#include <stdio.h>

int main(void) {
  /* n / 16777215.0f for all 2^24 numerators */
  const float d = 16777215.0f, rcp = 0x1.000002p-24f;
  if (rcp != 1.0f / d) { printf("rcp is not fl(1/d)\n"); return 1; }
  for (uint32_t n = 0; n < (1u << 24); ++n) {
    const float fn = (float)n;
    const float q = fn * rcp;
    const float fast = fmaf(fmaf(-q, d, fn), rcp, q);
    if (fast != fn / d) { printf("division differs at n=%u\n", n); return 1; }
  }
  /* r % m for all 16-bit r and all range widths 1..256 */
  for (uint32_t m = 1; m <= 256; ++m) {
    const uint32_t magic = m > 1 ? (uint32_t)((1ull << 32) / m) + 1u : 0u;
    for (uint32_t r = 0; r < 65536; ++r) {
      const uint32_t hi = (uint32_t)(((uint64_t)r * magic) >> 32);
      const uint32_t rem = m > 1 ? r - hi * m : 0u;
      if (rem != r % m) { printf("modulo differs at r=%u m=%u\n", r, m); return 1; }
    }
  }
  printf("exact arithmetic OK\n");
  return 0;
}
