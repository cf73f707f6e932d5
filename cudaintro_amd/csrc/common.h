// Shared declarations of the gfx950 GEMM library: context, status plumbing, vector types,
// narrowing conversions and the epilogue functors every kernel family uses.
#pragma once

#include <hip/hip_runtime.h>

#include <atomic>
#include <cstdint>
#include <cstdio>
#include <cstring>

#include "cigemm.h"

struct cigemmContext {
  uint32_t magic;
  int device;
  int num_cus;
  hipStream_t stream;
  const char* last_kernel;
  int last_tile_rows;  // rows of the output tile of the last tile-kernel launch, 0 otherwise
  int last_k_splits;   // K ranges of that launch
  int last_waves;      // wavefronts per workgroup of that launch
  int last_per_cu;     // workgroups of that launch resident per compute unit (1 or 2)
  int first_tile_rows; // when the call took two launches: rows and waves of the first, else 0
  int first_waves;
  char kernel_name[96];  // storage for names composed per call (last_kernel may point here)
  // A failure recorded while a launch was being prepared (a refused kernel attribute), reported
  // by check_launch as CIGEMM_STATUS_INTERNAL_ERROR; empty when there is none.
  char pending_error[160];
  int algo;  // cigemmAlgo_t; -1 = choose by shape
  // Device scratch of the split-K kernels, allocated once at create: `ws_partial_bytes` of
  // partial sums followed by `ws_counter_bytes` of arrival counters and `ws_swap_bytes` of
  // exchange words for two K ranges (both zero between calls).
  void* workspace;
  size_t ws_partial_bytes;
  size_t ws_counter_bytes;
  size_t ws_swap_bytes;
  // Set when a call on this handle ended in CIGEMM_STATUS_EXECUTION_FAILED: a split-K kernel
  // that did not run to its end may have left arrival counters or exchange words non-zero.
  // The next GEMM call clears both (a small kernel on the handle's stream) before it launches.
  int ws_dirty;
  // Measurement aid, set through the probe library only: with force_tile_mt in 1..4 the tile
  // kernel's launcher runs tiles of 64 * force_tile_mt rows over force_tile_splits K ranges
  // in place of its own plan; 0 = the launcher chooses.
  int force_tile_mt;
  int force_tile_splits;
  char last_error[256];
};

constexpr uint32_t kCtxMagic = 0xC16E3350u;

namespace cig {

// ---- status plumbing ------------------------------------------------------------------
cigemmStatus_t fail(cigemmContext* ctx, cigemmStatus_t st, const char* fmt, ...)
    __attribute__((format(printf, 3, 4)));
cigemmStatus_t check_launch(cigemmContext* ctx, const char* what);
// Name of a tile-kernel call from what the launcher recorded on the context, e.g.
// "i8_mfma_192x256x64_w4_ring4_nk_dequant" (tile rows x 256 columns x k elements per stage,
// waves per workgroup), "256+192" / "w4+w4" when two launches covered the columns.
void set_tile_kernel_name(cigemmContext* ctx, const char* dtype, int k_elems, const char* suffix,
                          bool splitk);
// Raises the dynamic-LDS limit of `kernel` to `bytes` once per device and template instance
// (`done` = that instance's bit mask of devices already set).  A refusal is recorded on the
// context and reported by check_launch; it returns false and the caller must not launch.
bool ensure_dynamic_lds(cigemmContext* ctx, const void* kernel, int bytes,
                        std::atomic<uint64_t>& done);

// ---- vector types ---------------------------------------------------------------------
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef int i32x2 __attribute__((ext_vector_type(2)));
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef int i32x16 __attribute__((ext_vector_type(16)));
typedef short i16x4 __attribute__((ext_vector_type(4)));
typedef short i16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

// ---- element conversions (device) -----------------------------------------------------
// bfloat16: the gfx950 conversion instruction (v_cvt_pk_bf16_f32) rounds to nearest even and
// quiets a NaN by setting mantissa bit 6 of the truncated pattern: on all 2^32 inputs it
// returns what the bit-pattern rule "u += 0x7FFF + ((u >> 16) & 1); NaN -> (u >> 16) | 0x40"
// returns.
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t f32x2_to_bf16_bits(float lo, float hi) {
  const f32x2 v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
}
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
  return __builtin_bit_cast(uint16_t, (__bf16)f);
}
__device__ __forceinline__ float bf16_bits_to_f32(uint16_t h) {
  return __builtin_bit_cast(float, (uint32_t)h << 16);
}
// binary16: the hardware conversion rounds to nearest even in the default FP mode.
__device__ __forceinline__ uint16_t f32_to_f16_bits(float f) {
  _Float16 h = (_Float16)f;
  return __builtin_bit_cast(uint16_t, h);
}
__device__ __forceinline__ uint32_t f32x2_to_f16_bits(float lo, float hi) {
  const f32x2 v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, f16x2));
}
__device__ __forceinline__ float f16_bits_to_f32(uint16_t h) {
  return (float)__builtin_bit_cast(_Float16, h);
}

// Element tags: how a 16-bit pattern is widened / narrowed.
struct BF16 {
  static __device__ __forceinline__ float widen(uint16_t h) { return bf16_bits_to_f32(h); }
  static __device__ __forceinline__ uint16_t narrow(float f) { return f32_to_bf16_bits(f); }
  static __device__ __forceinline__ uint32_t narrow2(float lo, float hi) {
    return f32x2_to_bf16_bits(lo, hi);
  }
};
struct F16 {
  static __device__ __forceinline__ float widen(uint16_t h) { return f16_bits_to_f32(h); }
  static __device__ __forceinline__ uint16_t narrow(float f) { return f32_to_f16_bits(f); }
  static __device__ __forceinline__ uint32_t narrow2(float lo, float hi) {
    return f32x2_to_f16_bits(lo, hi);
  }
};

// ---- epilogues --------------------------------------------------------------------------
// Each epilogue stores one accumulator for output element (row, col).

struct EpiBiasActF32 {  // fp32 linear layer: act(acc + bias[col])
  float* C;
  int64_t ldc;
  const float* bias;
  int relu;
  __device__ __forceinline__ void operator()(int64_t r, int64_t c, float acc) const {
    float v = bias ? __fadd_rn(acc, bias[c]) : acc;
    if (relu) v = fmaxf(0.0f, v);
    C[r * ldc + c] = v;
  }
};

struct EpiStoreF32 {  // fp32 GEMM
  float* C;
  int64_t ldc;
  __device__ __forceinline__ void operator()(int64_t r, int64_t c, float acc) const {
    C[r * ldc + c] = acc;
  }
};

template <typename E16>
struct EpiStore16 {  // fp16 / bf16 GEMM: one narrowing of the fp32 accumulator
  uint16_t* C;
  int64_t ldc;
  __device__ __forceinline__ void operator()(int64_t r, int64_t c, float acc) const {
    C[r * ldc + c] = E16::narrow(acc);
  }
};

struct EpiStoreI32 {  // int8 GEMM, raw accumulators
  int32_t* C;
  int64_t ldc;
  __device__ __forceinline__ void operator()(int64_t r, int64_t c, int32_t acc) const {
    C[r * ldc + c] = acc;
  }
};

// out = ((float)acc * sA) * sB, two separately rounded fp32 multiplies.  The float
// conversion of the accumulator rounds to nearest even (v_cvt_f32_i32).
template <bool OUT_BF16, bool DUMP_ACC>
struct EpiDequant {
  void* out;
  int64_t ldo;
  const float* sa;
  const float* sb;
  int sa_vec;  // 1: sa[row], 0: sa[0]
  int sb_vec;  // 1: sb[col], 0: sb[0]
  int32_t* acc_out;
  int64_t ldacc;
  __device__ __forceinline__ void operator()(int64_t r, int64_t c, int32_t acc) const {
    const float a = sa[sa_vec ? r : 0];
    const float b = sb[sb_vec ? c : 0];
    const float v = __fmul_rn(__fmul_rn((float)acc, a), b);
    if (OUT_BF16)
      static_cast<uint16_t*>(out)[r * ldo + c] = f32_to_bf16_bits(v);
    else
      static_cast<float*>(out)[r * ldo + c] = v;
    if (DUMP_ACC) acc_out[r * ldacc + c] = acc;
  }
};

// Bias + activation of the linear-layer entry point (bias may be null).
struct BiasAct {
  const float* bias;
  int relu;
};

struct DequantArgs {
  const float* sa;
  const float* sb;
  int sa_vec;
  int sb_vec;
  void* out;
  int out_bf16;
  int64_t ldo;
  int32_t* acc_out;
  int64_t ldacc;
};

// ---- kernel-family entry points (host side, defined in the per-family .hip files) ------
// Each returns true when it took the problem (launched), false when the shape or the
// alignment is outside what that family handles; the caller then falls through to the
// generic kernel.

// gemm_generic.hip: any shape, any alignment.
void launch_generic_f32(cigemmContext*, int64_t M, int64_t N, int64_t K, const float* A,
                        int64_t lda, const float* B, int64_t ldb, float* C, int64_t ldc,
                        const BiasAct* ba = nullptr);
// gemm_ragged.hip: any shape, any alignment, on the matrix cores.  False when
// the tile grid does not fit a launch (nothing launched).
bool launch_mfma_any_16(cigemmContext*, bool bf16, int64_t M, int64_t N, int64_t K,
                        const uint16_t* A, int64_t lda, const uint16_t* B, int64_t ldb,
                        uint16_t* C, int64_t ldc);
bool launch_mfma_any_f32(cigemmContext*, int64_t M, int64_t N, int64_t K, const float* A,
                         int64_t lda, const float* B, int64_t ldb, float* C, int64_t ldc,
                         const BiasAct* ba);
bool launch_mfma_any_i8(cigemmContext*, int64_t M, int64_t N, int64_t K, const int8_t* A,
                        int64_t lda, const int8_t* B, int64_t ldb, bool b_nk, int32_t* C,
                        int64_t ldc, const DequantArgs* dq);
void launch_generic_16(cigemmContext*, bool bf16, int64_t M, int64_t N, int64_t K,
                       const uint16_t* A, int64_t lda, const uint16_t* B, int64_t ldb,
                       uint16_t* C, int64_t ldc);
void launch_generic_i8(cigemmContext*, int64_t M, int64_t N, int64_t K, const int8_t* A,
                       int64_t lda, const int8_t* B, int64_t ldb, bool b_nk, int32_t* C,
                       int64_t ldc, const DequantArgs* dq);

// gemm_f32.hip: launch_f32_tile takes what the LDS-tiled kernel takes; launch_f32_mfma
// chooses between it and the small-tile kernel.  Both return false without launching when
// the shape is not theirs.
bool launch_f32_tile(cigemmContext*, int64_t M, int64_t N, int64_t K, const float* A,
                     int64_t lda, const float* B, int64_t ldb, float* C, int64_t ldc,
                     const BiasAct* ba = nullptr);
bool launch_f32_mfma(cigemmContext*, int64_t M, int64_t N, int64_t K, const float* A,
                     int64_t lda, const float* B, int64_t ldb, float* C, int64_t ldc,
                     const BiasAct* ba = nullptr);
// gemm_f32_small.hip: 32x32 tile per workgroup, k split over the waves.
bool f32_small_shape_ok(int64_t M, int64_t N, int64_t K, const float* A, int64_t lda);
void launch_f32_small(cigemmContext*, int64_t M, int64_t N, int64_t K, const float* A,
                      int64_t lda, const float* B, int64_t ldb, float* C, int64_t ldc,
                      const BiasAct* ba = nullptr);
// gemm_16b.hip
bool launch_16b_mfma(cigemmContext*, bool bf16, int64_t M, int64_t N, int64_t K,
                     const uint16_t* A, int64_t lda, const uint16_t* B, int64_t ldb,
                     uint16_t* C, int64_t ldc);
// gemm_i8.hip
bool launch_i8_mfma(cigemmContext*, int64_t M, int64_t N, int64_t K, const int8_t* A,
                    int64_t lda, const int8_t* B, int64_t ldb, bool b_nk, int32_t* C,
                    int64_t ldc, const DequantArgs* dq);
// gemm_skinny.hip
// Enqueues a kernel on the handle's stream that zeroes the arrival counters and the exchange
// words of the handle's workspace, and takes the dirty mark off the handle.
void clear_workspace(cigemmContext*);
bool launch_skinny_16(cigemmContext*, bool bf16, int64_t M, int64_t N, int64_t K,
                      const uint16_t* A, int64_t lda, const uint16_t* B, int64_t ldb,
                      uint16_t* C, int64_t ldc);
bool launch_skinny_i8(cigemmContext*, int64_t M, int64_t N, int64_t K, const int8_t* A,
                      int64_t lda, const int8_t* B, int64_t ldb, bool b_nk, int32_t* C,
                      int64_t ldc, const DequantArgs* dq);

}  // namespace cig
