// Epilogue functors shared by the MFMA kernel families.  Each call stores four consecutive
// columns col..col+3 of one output row.
#pragma once

#include "common.h"

namespace cig {

// Narrows four consecutive columns and stores them as one 8-byte piece.
template <typename E16>
struct EpiStore16x4 {
  uint16_t* C;
  int64_t ldc;
  __device__ __forceinline__ void operator()(int64_t r, int64_t c, float v0, float v1, float v2,
                                             float v3) const {
    u32x2 v;
    v[0] = (uint32_t)E16::narrow(v0) | ((uint32_t)E16::narrow(v1) << 16);
    v[1] = (uint32_t)E16::narrow(v2) | ((uint32_t)E16::narrow(v3) << 16);
    *reinterpret_cast<u32x2*>(C + r * ldc + c) = v;
  }
};

struct EpiStoreF32x4 {
  float* C;
  int64_t ldc;
  __device__ __forceinline__ void operator()(int64_t r, int64_t c, float v0, float v1, float v2,
                                             float v3) const {
    *reinterpret_cast<f32x4*>(C + r * ldc + c) = f32x4{v0, v1, v2, v3};
  }
};

struct EpiStoreI32x4 {
  int32_t* C;
  int64_t ldc;
  __device__ __forceinline__ void operator()(int64_t r, int64_t c, int32_t v0, int32_t v1,
                                             int32_t v2, int32_t v3) const {
    i32x4 v = {v0, v1, v2, v3};
    *reinterpret_cast<i32x4*>(C + r * ldc + c) = v;
  }
};

// out = ((float)acc * sA[row]) * sB[col]: two separately rounded fp32 multiplies, then an
// optional round-to-nearest-even narrowing to bf16.  Four consecutive columns per call.
template <bool OUT_BF16, bool DUMP_ACC>
struct EpiDequantX4 {
  void* out;
  int64_t ldo;
  const float* sa;
  const float* sb;
  int sa_vec, sb_vec;
  int32_t* acc_out;
  int64_t ldacc;
  __device__ __forceinline__ void operator()(int64_t r, int64_t c, int32_t v0, int32_t v1,
                                             int32_t v2, int32_t v3) const {
    const float a = sa[sa_vec ? r : 0];
    f32x4 b;
    if (sb_vec)
      b = *reinterpret_cast<const f32x4*>(sb + c);
    else
      b = f32x4{sb[0], sb[0], sb[0], sb[0]};
    float o[4];
    o[0] = __fmul_rn(__fmul_rn((float)v0, a), b[0]);
    o[1] = __fmul_rn(__fmul_rn((float)v1, a), b[1]);
    o[2] = __fmul_rn(__fmul_rn((float)v2, a), b[2]);
    o[3] = __fmul_rn(__fmul_rn((float)v3, a), b[3]);
    if (OUT_BF16) {
      u32x2 p;
      p[0] = (uint32_t)f32_to_bf16_bits(o[0]) | ((uint32_t)f32_to_bf16_bits(o[1]) << 16);
      p[1] = (uint32_t)f32_to_bf16_bits(o[2]) | ((uint32_t)f32_to_bf16_bits(o[3]) << 16);
      *reinterpret_cast<u32x2*>(static_cast<uint16_t*>(out) + r * ldo + c) = p;
    } else {
      *reinterpret_cast<f32x4*>(static_cast<float*>(out) + r * ldo + c) =
          f32x4{o[0], o[1], o[2], o[3]};
    }
    if (DUMP_ACC) {
      i32x4 v = {v0, v1, v2, v3};
      *reinterpret_cast<i32x4*>(acc_out + r * ldacc + c) = v;
    }
  }
};

}  // namespace cig
