// Epilogue functors shared by the MFMA kernel families.  An epilogue turns four consecutive
// accumulators of one output row (columns col..col+3) into output bits:
//   load_row(row)            what the epilogue needs per output row (a scale), fetched once;
//   load_cols(col)           what it needs for the four columns col..col+3 (scales, bias);
//   pack(rowv, colv, v0..v3) the 4 output elements as raw bits (u32x2 for 16-bit outputs,
//                            u32x4 for 32-bit ones) from those; no memory is touched;
//   pack(row, col, v0..v3)   the same with both fetched on the spot;
//   side(row, col, v0..v3)   any second output of the same quad (the accumulator dump);
//   out_row(row)             byte address of column 0 of that output row;
//   operator()               pack + direct store (used where rows are not staged in LDS);
//   shift_cols(c)            the same epilogue for the sub-problem starting at column c.
// An epilogue whose row or column operand can be one word for the whole matrix (a per-tensor
// scale) may declare `static constexpr bool HAS_UNIFORM_MODE = true` and give
//   row_word(), col_word()           the address of that word (always readable);
//   row_uniform(), col_uniform()     whether this call uses it;
//   row_from_word(w), cols_from_word(w)   what load_row / load_cols would return, from it.
// A kernel can then read the word once, with a scalar load, long before the epilogue.
#pragma once

#include <type_traits>

#include "common.h"

namespace cig {

struct EpiNothing {};

// Narrows four consecutive columns and stores them as one 8-byte piece.
template <typename E16>
struct EpiStore16x4 {
  uint16_t* C;
  int64_t ldc;
  static constexpr int OUT_BYTES = 2;
  typedef EpiNothing row_t;
  typedef EpiNothing col_t;
  __device__ __forceinline__ row_t load_row(int64_t) const { return row_t{}; }
  __device__ __forceinline__ col_t load_cols(int64_t) const { return col_t{}; }
  __device__ __forceinline__ u32x2 pack(row_t, col_t, float v0, float v1, float v2,
                                        float v3) const {
    return pack(0, 0, v0, v1, v2, v3);
  }
  __device__ __forceinline__ u32x2 pack(int64_t, int64_t, float v0, float v1, float v2,
                                        float v3) const {
    u32x2 v;
    v[0] = E16::narrow2(v0, v1);
    v[1] = E16::narrow2(v2, v3);
    return v;
  }
  __device__ __forceinline__ char* out_row(int64_t r) const {
    return reinterpret_cast<char*>(C + r * ldc);
  }
  __device__ __forceinline__ void operator()(int64_t r, int64_t c, float v0, float v1, float v2,
                                             float v3) const {
    *reinterpret_cast<u32x2*>(C + r * ldc + c) = pack(r, c, v0, v1, v2, v3);
  }
  // two columns (c even): one 4-byte store
  __device__ __forceinline__ void pair(int64_t r, int64_t c, float v0, float v1) const {
    *reinterpret_cast<uint32_t*>(C + r * ldc + c) = E16::narrow2(v0, v1);
  }
  __device__ __forceinline__ void side(int64_t, int64_t, float, float, float, float) const {}
  EpiStore16x4 shift_cols(int64_t c0) const { return EpiStore16x4{C + c0, ldc}; }
};

struct EpiStoreF32x4 {
  float* C;
  int64_t ldc;
  static constexpr int OUT_BYTES = 4;
  typedef EpiNothing row_t;
  typedef EpiNothing col_t;
  __device__ __forceinline__ row_t load_row(int64_t) const { return row_t{}; }
  __device__ __forceinline__ col_t load_cols(int64_t) const { return col_t{}; }
  __device__ __forceinline__ u32x4 pack(row_t, col_t, float v0, float v1, float v2,
                                        float v3) const {
    return pack(0, 0, v0, v1, v2, v3);
  }
  __device__ __forceinline__ u32x4 pack(int64_t, int64_t, float v0, float v1, float v2,
                                        float v3) const {
    return __builtin_bit_cast(u32x4, f32x4{v0, v1, v2, v3});
  }
  __device__ __forceinline__ char* out_row(int64_t r) const {
    return reinterpret_cast<char*>(C + r * ldc);
  }
  __device__ __forceinline__ void operator()(int64_t r, int64_t c, float v0, float v1, float v2,
                                             float v3) const {
    *reinterpret_cast<f32x4*>(C + r * ldc + c) = f32x4{v0, v1, v2, v3};
  }
  __device__ __forceinline__ void side(int64_t, int64_t, float, float, float, float) const {}
  EpiStoreF32x4 shift_cols(int64_t c0) const { return EpiStoreF32x4{C + c0, ldc}; }
};

// fp32 linear layer: act(acc + bias[col]); RELU and HAS_BIAS are compile-time.
template <bool HAS_BIAS, bool RELU>
struct EpiBiasActF32x4 {
  float* C;
  int64_t ldc;
  const float* bias;
  static constexpr int OUT_BYTES = 4;
  typedef EpiNothing row_t;
  typedef f32x4 col_t;  // bias of the four columns
  __device__ __forceinline__ row_t load_row(int64_t) const { return row_t{}; }
  __device__ __forceinline__ col_t load_cols(int64_t c) const {
    if (HAS_BIAS) return *reinterpret_cast<const f32x4*>(bias + c);
    return f32x4{0.0f, 0.0f, 0.0f, 0.0f};
  }
  __device__ __forceinline__ u32x4 pack(row_t, col_t b, float v0, float v1, float v2,
                                        float v3) const {
    f32x4 v = {v0, v1, v2, v3};
    if (HAS_BIAS) {
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] = __fadd_rn(v[e], b[e]);
    }
    if (RELU) {
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] = fmaxf(0.0f, v[e]);
    }
    return __builtin_bit_cast(u32x4, v);
  }
  __device__ __forceinline__ u32x4 pack(int64_t r, int64_t c, float v0, float v1, float v2,
                                        float v3) const {
    return pack(load_row(r), load_cols(c), v0, v1, v2, v3);
  }
  __device__ __forceinline__ char* out_row(int64_t r) const {
    return reinterpret_cast<char*>(C + r * ldc);
  }
  __device__ __forceinline__ void side(int64_t, int64_t, float, float, float, float) const {}
  __device__ __forceinline__ void operator()(int64_t r, int64_t c, float v0, float v1, float v2,
                                             float v3) const {
    *reinterpret_cast<u32x4*>(C + r * ldc + c) = pack(r, c, v0, v1, v2, v3);
  }
  EpiBiasActF32x4 shift_cols(int64_t c0) const {
    return EpiBiasActF32x4{C + c0, ldc, HAS_BIAS ? bias + c0 : bias};
  }
};

struct EpiStoreI32x4 {
  int32_t* C;
  int64_t ldc;
  static constexpr int OUT_BYTES = 4;
  typedef EpiNothing row_t;
  typedef EpiNothing col_t;
  __device__ __forceinline__ row_t load_row(int64_t) const { return row_t{}; }
  __device__ __forceinline__ col_t load_cols(int64_t) const { return col_t{}; }
  __device__ __forceinline__ u32x4 pack(row_t, col_t, int32_t v0, int32_t v1, int32_t v2,
                                        int32_t v3) const {
    return pack(0, 0, v0, v1, v2, v3);
  }
  __device__ __forceinline__ u32x4 pack(int64_t, int64_t, int32_t v0, int32_t v1, int32_t v2,
                                        int32_t v3) const {
    return __builtin_bit_cast(u32x4, i32x4{v0, v1, v2, v3});
  }
  __device__ __forceinline__ char* out_row(int64_t r) const {
    return reinterpret_cast<char*>(C + r * ldc);
  }
  __device__ __forceinline__ void operator()(int64_t r, int64_t c, int32_t v0, int32_t v1,
                                             int32_t v2, int32_t v3) const {
    i32x4 v = {v0, v1, v2, v3};
    *reinterpret_cast<i32x4*>(C + r * ldc + c) = v;
  }
  __device__ __forceinline__ void side(int64_t, int64_t, int32_t, int32_t, int32_t, int32_t) const {}
  EpiStoreI32x4 shift_cols(int64_t c0) const { return EpiStoreI32x4{C + c0, ldc}; }
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
  static constexpr int OUT_BYTES = OUT_BF16 ? 2 : 4;
  static constexpr bool REGISTER_HEAVY = DUMP_ACC;  // 256-row tile: stay on the four-wave form
  typedef typename std::conditional<OUT_BF16, u32x2, u32x4>::type packed_t;
  typedef float row_t;   // scale of the row
  typedef f32x4 col_t;   // scales of the four columns
  static constexpr bool HAS_UNIFORM_MODE = true;
  __device__ __forceinline__ const float* row_word() const { return sa; }
  __device__ __forceinline__ const float* col_word() const { return sb; }
  __device__ __forceinline__ bool row_uniform() const { return !sa_vec; }
  __device__ __forceinline__ bool col_uniform() const { return !sb_vec; }
  __device__ __forceinline__ row_t row_from_word(float w) const { return w; }
  __device__ __forceinline__ col_t cols_from_word(float w) const { return f32x4{w, w, w, w}; }
  __device__ __forceinline__ row_t load_row(int64_t r) const { return sa[sa_vec ? r : 0]; }
  __device__ __forceinline__ col_t load_cols(int64_t c) const {
    if (sb_vec) return *reinterpret_cast<const f32x4*>(sb + c);
    const float b0 = sb[0];
    return f32x4{b0, b0, b0, b0};
  }
  __device__ __forceinline__ packed_t pack(row_t a, col_t b, int32_t v0, int32_t v1, int32_t v2,
                                           int32_t v3) const {
    float o[4];
    o[0] = __fmul_rn(__fmul_rn((float)v0, a), b[0]);
    o[1] = __fmul_rn(__fmul_rn((float)v1, a), b[1]);
    o[2] = __fmul_rn(__fmul_rn((float)v2, a), b[2]);
    o[3] = __fmul_rn(__fmul_rn((float)v3, a), b[3]);
    if constexpr (OUT_BF16) {
      u32x2 p;
      p[0] = f32x2_to_bf16_bits(o[0], o[1]);
      p[1] = f32x2_to_bf16_bits(o[2], o[3]);
      return p;
    } else {
      return __builtin_bit_cast(u32x4, f32x4{o[0], o[1], o[2], o[3]});
    }
  }
  __device__ __forceinline__ packed_t pack(int64_t r, int64_t c, int32_t v0, int32_t v1,
                                           int32_t v2, int32_t v3) const {
    return pack(load_row(r), load_cols(c), v0, v1, v2, v3);
  }
  __device__ __forceinline__ char* out_row(int64_t r) const {
    return static_cast<char*>(out) + r * ldo * OUT_BYTES;
  }
  __device__ __forceinline__ void side(int64_t r, int64_t c, int32_t v0, int32_t v1, int32_t v2,
                                       int32_t v3) const {
    if (DUMP_ACC) {
      i32x4 v = {v0, v1, v2, v3};
      *reinterpret_cast<i32x4*>(acc_out + r * ldacc + c) = v;
    }
  }
  __device__ __forceinline__ void operator()(int64_t r, int64_t c, int32_t v0, int32_t v1,
                                             int32_t v2, int32_t v3) const {
    *reinterpret_cast<packed_t*>(out_row(r) + c * OUT_BYTES) = pack(r, c, v0, v1, v2, v3);
    side(r, c, v0, v1, v2, v3);
  }
  EpiDequantX4 shift_cols(int64_t c0) const {
    EpiDequantX4 e = *this;
    e.out = OUT_BF16 ? static_cast<void*>(static_cast<uint16_t*>(out) + c0)
                     : static_cast<void*>(static_cast<float*>(out) + c0);
    if (sb_vec) e.sb = sb + c0;
    if (DUMP_ACC) e.acc_out = acc_out + c0;
    return e;
  }
};

}  // namespace cig
