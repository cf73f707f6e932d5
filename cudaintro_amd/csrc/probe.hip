// Measurement aid: a register-resident matrix-core loop (no memory traffic in the loop), one
// wave per SIMD on every compute unit, to show what the chip sustains at the clock it
// actually holds under this load.  Sustained rate depends on the operand data (the chip is
// power limited), so the probe runs on constant or on pseudo-random operand bits.
#include "common.h"

namespace cig {
namespace {

constexpr int PROBE_UNROLL = 12;  // independent accumulators per wave (no register spills)

__device__ __forceinline__ uint32_t mix32(uint32_t x) {
  x ^= x >> 16; x *= 0x7feb352du; x ^= x >> 15; x *= 0x846ca68bu; x ^= x >> 16;
  return x;
}

// KIND 0: bf16 32x32x16, 1: f16 32x32x16, 2: int8 32x32x32, 3: bf16 16x16x32, 4: f16 16x16x32,
// 5: int8 16x16x64, 6: fp32 32x32x2.
template <int KIND>
__global__ __launch_bounds__(256, 1) void mfma_probe_kernel(float* __restrict__ out, int iters,
                                                            int random_bits) {
  // four operand pairs, cycled through the unrolled MFMAs so that consecutive instructions
  // see different bits on the random setting
  u32x4 a[4], b[4];
#pragma unroll
  for (int s = 0; s < 4; ++s)
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      uint32_t xa = mix32((threadIdx.x * 8 + s * 2) * 4 + e + 1);
      uint32_t xb = mix32((threadIdx.x * 8 + s * 2 + 1) * 4 + e + 1);
      if (!random_bits) xa = xb = 0;
      if (KIND == 0 || KIND == 3) {  // +-[1,2) in bf16: random sign and mantissa
        xa = (xa & 0x807f807fu) | 0x3f803f80u;
        xb = (xb & 0x807f807fu) | 0x3f803f80u;
      } else if (KIND == 1 || KIND == 4) {  // +-[1,2) in fp16
        xa = (xa & 0x83ff83ffu) | 0x3c003c00u;
        xb = (xb & 0x83ff83ffu) | 0x3c003c00u;
      } else if (KIND == 6) {  // +-[1,2) in fp32
        xa = (xa & 0x807fffffu) | 0x3f800000u;
        xb = (xb & 0x807fffffu) | 0x3f800000u;
      } else if (!random_bits) {
        xa = xb = 0x01010101u;
      }
      a[s][e] = xa;
      b[s][e] = xb;
    }
  f32x16 facc[PROBE_UNROLL];
  i32x16 iacc[PROBE_UNROLL];
  f32x4 facc4[PROBE_UNROLL];
  i32x4 iacc4[PROBE_UNROLL];
#pragma unroll
  for (int i = 0; i < PROBE_UNROLL; ++i)
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      facc4[i][e] = 0.0f;
      iacc4[i][e] = 0;
    }
#pragma unroll
  for (int i = 0; i < PROBE_UNROLL; ++i)
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      facc[i][e] = 0.0f;
      iacc[i][e] = 0;
    }
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < PROBE_UNROLL; ++i) {
      const u32x4 x = a[i & 3], y = b[(i + (i >> 2)) & 3];
      if (KIND == 0)
        facc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, x),
                                                          __builtin_bit_cast(bf16x8, y), facc[i], 0, 0, 0);
      else if (KIND == 1)
        facc[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, x),
                                                         __builtin_bit_cast(f16x8, y), facc[i], 0, 0, 0);
      else if (KIND == 2)
        iacc[i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(__builtin_bit_cast(i32x4, x),
                                                        __builtin_bit_cast(i32x4, y), iacc[i], 0, 0, 0);
      else if (KIND == 3)
        facc4[i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, x),
                                                           __builtin_bit_cast(bf16x8, y), facc4[i], 0, 0, 0);
      else if (KIND == 4)
        facc4[i] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, x),
                                                          __builtin_bit_cast(f16x8, y), facc4[i], 0, 0, 0);
      else if (KIND == 6)
        facc[i] = __builtin_amdgcn_mfma_f32_32x32x2f32(__builtin_bit_cast(float, x[(i & 3) ^ 1]),
                                                       __builtin_bit_cast(float, y[i & 3]), facc[i], 0, 0, 0);
      else
        iacc4[i] = __builtin_amdgcn_mfma_i32_16x16x64_i8(__builtin_bit_cast(i32x4, x),
                                                         __builtin_bit_cast(i32x4, y), iacc4[i], 0, 0, 0);
    }
  }
  float s = 0.0f;
#pragma unroll
  for (int i = 0; i < PROBE_UNROLL; ++i)
#pragma unroll
    for (int e = 0; e < 16; ++e) s += facc[i][e] + (float)iacc[i][e] + facc4[i][e & 3] + (float)iacc4[i][e & 3];
  out[blockIdx.x * 256 + threadIdx.x] = s;
}

}  // namespace
}  // namespace cig

using namespace cig;

extern "C" cigemmStatus_t cigemm_probe_mfma(cigemmHandle_t h, int kind, int random_bits, int iters,
                                            int64_t* ops_per_launch) {
  if (!h || h->magic != kCtxMagic) return CIGEMM_STATUS_NOT_INITIALIZED;
  if (kind < 0 || kind > 6 || iters <= 0 || iters > (1 << 24))
    return fail(h, CIGEMM_STATUS_INVALID_VALUE, "cigemm_probe_mfma: kind %d, iters %d", kind, iters);
  const int grid = h->num_cus > 0 ? h->num_cus : 256;
  if (!h->workspace || (size_t)grid * 256 * sizeof(float) > h->ws_partial_bytes)
    return fail(h, CIGEMM_STATUS_ALLOC_FAILED, "cigemm_probe_mfma: workspace too small");
  float* out = static_cast<float*>(h->workspace);
  if (kind == 0)
    hipLaunchKernelGGL(mfma_probe_kernel<0>, dim3(grid), dim3(256), 0, h->stream, out, iters, random_bits);
  else if (kind == 1)
    hipLaunchKernelGGL(mfma_probe_kernel<1>, dim3(grid), dim3(256), 0, h->stream, out, iters, random_bits);
  else if (kind == 2)
    hipLaunchKernelGGL(mfma_probe_kernel<2>, dim3(grid), dim3(256), 0, h->stream, out, iters, random_bits);
  else if (kind == 3)
    hipLaunchKernelGGL(mfma_probe_kernel<3>, dim3(grid), dim3(256), 0, h->stream, out, iters, random_bits);
  else if (kind == 4)
    hipLaunchKernelGGL(mfma_probe_kernel<4>, dim3(grid), dim3(256), 0, h->stream, out, iters, random_bits);
  else if (kind == 5)
    hipLaunchKernelGGL(mfma_probe_kernel<5>, dim3(grid), dim3(256), 0, h->stream, out, iters, random_bits);
  else
    hipLaunchKernelGGL(mfma_probe_kernel<6>, dim3(grid), dim3(256), 0, h->stream, out, iters, random_bits);
  if (ops_per_launch)
    *ops_per_launch = (int64_t)grid * 4 * (int64_t)iters * PROBE_UNROLL *
                      (kind == 2 ? 65536 : kind == 6 ? 4096 : kind == 5 ? 32768 : kind >= 3 ? 16384 : 32768);
  h->last_kernel = "mfma_probe";
  return check_launch(h, "cigemm_probe_mfma");
}
