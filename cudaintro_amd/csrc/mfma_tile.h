// The LDS-tiled MFMA GEMM kernel shared by the bf16, fp16 and int8 families.
//
// Workgroup = 256 lanes = 4 waves (2 x 2); macro tile 256 (m) x 256 (n) x 128 BYTES of k
// (64 halves or 128 int8).  Each wave owns a 128 x 128 block = 4 x 4 MFMA tiles of 32 x 32
// = 256 accumulators per lane.  Both operand tiles are 32 KiB; two stages are kept in LDS.
//
// A tile  [256 m][128 B of k], as in memory.  16-byte chunk c of row r lives at
//         r*128 + ((c ^ fA(r)) << 4): the 16-byte fragment reads of 32 consecutive rows
//         then spread over all banks.
// B tile  one of
//   NK    [256 n][128 B of k]  (weights, k contiguous): same geometry and reads as A;
//   KN16  [64 k][256 n] halves, KN8 [128 k][256 n] bytes (n contiguous, as C = A.B stores
//         B).  The MFMA wants k contiguous per lane, so fragments come from the transposing
//         LDS reads ds_read_b64_tr_b16 / _tr_b8: within 16 lanes, lane i supplies the
//         address of 8 bytes of row k0 + i/4 (i/2 for bytes) and receives the 4 (8)
//         k-values of column n0 + i.  Chunks are XOR-swizzled by k so that the rows one
//         instruction touches fall in different banks.
//
// The MFMA is issued with the B fragment as its first operand and the A fragment as its
// second, so it yields the transposed 32 x 32 block: lane l holds, for the single output
// row m = l%32, columns 8q + 4(l/32) + e (q, e = 0..3) in accumulator 4q+e, i.e. four
// consecutive columns per quad, which the epilogue stores as one piece of a row of C.
#pragma once

#include <type_traits>

#include "common.h"

namespace cig {
namespace tile {

constexpr int BM = 256, BN = 256;
constexpr int KB = 128;                    // bytes of k per stage, per row
constexpr int OPERAND_BYTES = 256 * KB;    // 32 KiB, either operand
constexpr int STAGE_BYTES = 2 * OPERAND_BYTES;
constexpr int LDS_BYTES = 2 * STAGE_BYTES;  // 128 KiB of the 160 KiB

typedef __attribute__((address_space(3))) i16x4 lds_i16x4;
typedef __attribute__((address_space(3))) i32x2 lds_i32x2;

// ---- A-like tile: [256 rows][8 chunks] ----------------------------------------------------
__device__ __forceinline__ int rowmajor_off(int r, int c) {
  const int f = ((r >> 1) & 7) ^ ((r & 1) << 2);
  return r * KB + ((c ^ f) << 4);
}

enum BMode { B_NK = 0, B_KN16 = 1, B_KN8 = 2 };

template <int MODE>
struct BTile;

// Weights N x K: identical to the A tile.
template <>
struct BTile<B_NK> {
  // lane t loads chunk t%8 of row t/8 + 32 i
  static __device__ __forceinline__ int ld_row(int t, int i) { return (t >> 3) + 32 * i; }
  static __device__ __forceinline__ int ld_chunk(int t) { return t & 7; }
  static __device__ __forceinline__ int off(int r, int c) { return rowmajor_off(r, c); }
  // global element offset of (tile row r = n, chunk c) at k byte offset kbyte0
  static __device__ __forceinline__ int64_t gofs(int r, int c, int64_t ld, int64_t n0,
                                                 int64_t kbyte0) {
    return (n0 + r) * ld + kbyte0 + c * 16;  // bytes == elements (int8)
  }
  // fragment for column tile j of wave column wn, k-step kk
  static __device__ __forceinline__ u32x4 frag(const char* sb, int wn, int j, int kk, int l) {
    const int r = wn * 128 + 32 * j + (l & 31);
    return *reinterpret_cast<const u32x4*>(sb + rowmajor_off(r, 2 * kk + (l >> 5)));
  }
};

// K x N halves: [64 k][32 chunks of 8 halves].
template <>
struct BTile<B_KN16> {
  static __device__ __forceinline__ int ld_row(int t, int i) { return (t >> 5) + 8 * i; }
  static __device__ __forceinline__ int ld_chunk(int t) { return t & 31; }
  static __device__ __forceinline__ int off(int k, int c) {
    const int k3 = k & 3;
    const int g = (k3 << 2) | ((((k3 >> 1) ^ k3) & 1) << 1);
    return k * 512 + ((c ^ g) << 4);
  }
  static __device__ __forceinline__ u32x4 frag(const char* sb, int wn, int j, int kk, int l) {
    const int k_lo = 16 * kk + 8 * (l >> 5) + ((l & 15) >> 2);
    const int n = wn * 128 + 32 * j + 16 * ((l >> 4) & 1) + 4 * (l & 3);
    const int sub = ((n >> 2) & 1) * 8;
    i16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4*)(sb + off(k_lo, n >> 3) + sub));
    i16x4 hi =
        __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4*)(sb + off(k_lo + 4, n >> 3) + sub));
    i16x8 both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    return __builtin_bit_cast(u32x4, both);
  }
};

// K x N bytes: [128 k][16 chunks of 16 bytes].
template <>
struct BTile<B_KN8> {
  static __device__ __forceinline__ int ld_row(int t, int i) { return (t >> 4) + 16 * i; }
  static __device__ __forceinline__ int ld_chunk(int t) { return t & 15; }
  static __device__ __forceinline__ int off(int k, int c) {
    const int g = ((k & 7) << 1) | (((k >> 2) ^ (k >> 4)) & 1);
    return k * 256 + ((c ^ g) << 4);
  }
  static __device__ __forceinline__ u32x4 frag(const char* sb, int wn, int j, int kk, int l) {
    const int k_lo = 32 * kk + 16 * (l >> 5) + ((l & 15) >> 1);
    const int n = wn * 128 + 32 * j + 16 * ((l >> 4) & 1) + 8 * (l & 1);
    const int sub = ((n >> 3) & 1) * 8;
    i32x2 lo = __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_i32x2*)(sb + off(k_lo, n >> 4) + sub));
    i32x2 hi =
        __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_i32x2*)(sb + off(k_lo + 8, n >> 4) + sub));
    i32x4 both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3);
    return __builtin_bit_cast(u32x4, both);
  }
};

// ---- arithmetic traits ----------------------------------------------------------------------
struct MathBF16 {
  typedef f32x16 acc_t;
  typedef float scalar_t;
  static constexpr int ELEM_BYTES = 2;
  static __device__ __forceinline__ acc_t mfma(u32x4 first, u32x4 second, acc_t acc) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, first),
                                                   __builtin_bit_cast(bf16x8, second), acc, 0, 0,
                                                   0);
  }
};
struct MathF16 {
  typedef f32x16 acc_t;
  typedef float scalar_t;
  static constexpr int ELEM_BYTES = 2;
  static __device__ __forceinline__ acc_t mfma(u32x4 first, u32x4 second, acc_t acc) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, first),
                                                  __builtin_bit_cast(f16x8, second), acc, 0, 0, 0);
  }
};
struct MathI8 {
  typedef i32x16 acc_t;
  typedef int32_t scalar_t;
  static constexpr int ELEM_BYTES = 1;
  static __device__ __forceinline__ acc_t mfma(u32x4 first, u32x4 second, acc_t acc) {
    return __builtin_amdgcn_mfma_i32_32x32x32_i8(__builtin_bit_cast(i32x4, first),
                                                 __builtin_bit_cast(i32x4, second), acc, 0, 0, 0);
  }
};

// Maps the hardware workgroup id to an output tile.  Workgroups are handed to the 8 XCDs
// round-robin; the remap gives each XCD a contiguous range of logical ids, and logical ids
// walk the tile grid in column-major groups of GROUP_M tile rows, so the tiles resident on
// one XCD at a time share A row panels and B column panels in that XCD's L2.
__device__ __forceinline__ void tile_of_workgroup(int tiles_m, int tiles_n, int& tm, int& tn) {
  constexpr int XCDS = 8, GROUP_M = 8;
  const int nwg = tiles_m * tiles_n;
  const int pid = blockIdx.x;
  const int xcd = pid % XCDS, local = pid / XCDS;
  const int base = nwg / XCDS, rem = nwg % XCDS;
  const int wg = xcd * base + (xcd < rem ? xcd : rem) + local;
  const int per_group = GROUP_M * tiles_n;
  const int group = wg / per_group;
  const int first_m = group * GROUP_M;
  const int gsize = (tiles_m - first_m) < GROUP_M ? (tiles_m - first_m) : GROUP_M;
  const int in_group = wg % per_group;
  tm = first_m + in_group % gsize;
  tn = in_group / gsize;
}

// Epi: __device__ void operator()(int64_t row, int64_t col, scalar v0, v1, v2, v3) stores the
// four consecutive columns col..col+3 of one output row.
//
// A, B are byte pointers; lda/ldb are in BYTES.  K_bytes = K * ELEM_BYTES is a multiple of
// 128, M and N multiples of 256, all rows 16-byte aligned (the launcher checks).
template <typename Math, int BMODE, typename Epi>
__global__ __launch_bounds__(256, 1) void mfma_tile_kernel(int tiles_m, int tiles_n, int KT,
                                                           const char* __restrict__ A,
                                                           int64_t lda,
                                                           const char* __restrict__ B,
                                                           int64_t ldb, Epi epi) {
  typedef typename Math::acc_t acc_t;
  typedef BTile<BMODE> BT;
  extern __shared__ __attribute__((aligned(1024))) char lds[];
  const int t = threadIdx.x;
  const int l = t & 63;
  const int w = t >> 6;
  const int wm = w >> 1, wn = w & 1;

  int tm, tn;
  tile_of_workgroup(tiles_m, tiles_n, tm, tn);
  const int64_t m0 = (int64_t)tm * BM, n0 = (int64_t)tn * BN;

  // ---- global -> register staging: 8 + 8 16-byte loads per lane per stage -------------------
  const int a_chunk = t & 7;
  const char* a_src = A + (m0 + (t >> 3)) * lda + a_chunk * 16;
  const int64_t a_step = 32 * lda;  // between this lane's 8 rows
  const char* b_src;
  int64_t b_step, b_kstep;  // between this lane's 8 rows; between stages
  if (BMODE == B_NK) {
    b_src = B + (n0 + BT::ld_row(t, 0)) * ldb + BT::ld_chunk(t) * 16;
    b_step = 32 * ldb;
    b_kstep = KB;
  } else {
    b_src = B + (int64_t)BT::ld_row(t, 0) * ldb + n0 * Math::ELEM_BYTES + BT::ld_chunk(t) * 16;
    b_step = (int64_t)(BT::ld_row(t, 1) - BT::ld_row(t, 0)) * ldb;
    b_kstep = (int64_t)(KB / Math::ELEM_BYTES) * ldb;
  }
  int a_dst[8], b_dst[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    a_dst[i] = rowmajor_off((t >> 3) + 32 * i, a_chunk);
    b_dst[i] = OPERAND_BYTES + BT::off(BT::ld_row(t, i), BT::ld_chunk(t));
  }
  u32x4 a_stage[8], b_stage[8];

  auto load_global = [&](int kt) {
    const char* ap = a_src + (int64_t)kt * KB;
    const char* bp = b_src + (int64_t)kt * b_kstep;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      a_stage[i] = *reinterpret_cast<const u32x4*>(ap + i * a_step);
      b_stage[i] = *reinterpret_cast<const u32x4*>(bp + i * b_step);
    }
  };
  auto store_lds = [&](int buf) {
    char* base = lds + buf * STAGE_BYTES;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      *reinterpret_cast<u32x4*>(base + a_dst[i]) = a_stage[i];
      *reinterpret_cast<u32x4*>(base + b_dst[i]) = b_stage[i];
    }
  };

  const int a_frag_row = wm * 128 + (l & 31);
  const int g = l >> 5;

  acc_t acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0;

  load_global(0);
  store_lds(0);
  __syncthreads();

  for (int kt = 0; kt < KT; ++kt) {
    const int buf = kt & 1;
    if (kt + 1 < KT) load_global(kt + 1);
    const char* sa = lds + buf * STAGE_BYTES;
    const char* sb = sa + OPERAND_BYTES;
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
      u32x4 af[4], bf[4];
#pragma unroll
      for (int i = 0; i < 4; ++i)
        af[i] = *reinterpret_cast<const u32x4*>(sa + rowmajor_off(a_frag_row + 32 * i, 2 * kk + g));
#pragma unroll
      for (int j = 0; j < 4; ++j) bf[j] = BT::frag(sb, wn, j, kk, l);
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = Math::mfma(bf[j], af[i], acc[i][j]);
    }
    if (kt + 1 < KT) store_lds(buf ^ 1);
    __syncthreads();
  }

  // acc[i][j][4q+e] = C[m0 + wm*128 + 32i + l%32][n0 + wn*128 + 32j + 8q + 4g + e]
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int64_t row = m0 + wm * 128 + 32 * i + (l & 31);
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int q = 0; q < 4; ++q)
        epi(row, n0 + wn * 128 + 32 * j + 8 * q + 4 * g, acc[i][j][4 * q + 0],
            acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]);
  }
}

template <typename Math, int BMODE, typename Epi>
void launch_tile(cigemmContext* ctx, int64_t M, int64_t N, int64_t K_bytes, const void* A,
                 int64_t lda_bytes, const void* B, int64_t ldb_bytes, const Epi& epi) {
  auto kern = mfma_tile_kernel<Math, BMODE, Epi>;
  static int attr_device = -1;  // one per template instance
  if (attr_device != ctx->device) {
    (void)hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize,
                              LDS_BYTES);
    attr_device = ctx->device;
  }
  const int tiles_m = (int)(M / BM), tiles_n = (int)(N / BN);
  hipLaunchKernelGGL(kern, dim3((unsigned)(tiles_m * tiles_n)), dim3(256), LDS_BYTES, ctx->stream,
                     tiles_m, tiles_n, (int)(K_bytes / KB), static_cast<const char*>(A),
                     lda_bytes, static_cast<const char*>(B), ldb_bytes, epi);
}

// Shape / alignment gate shared by the families (sizes in elements, elem = bytes each).
inline bool tile_shape_ok(int64_t M, int64_t N, int64_t K, int elem, const void* A, int64_t lda,
                          const void* B, int64_t ldb) {
  if (M <= 0 || N <= 0 || K <= 0) return false;
  if (M % BM || N % BN || (K * elem) % KB) return false;
  if ((lda * elem) % 16 || (ldb * elem) % 16) return false;
  if (((uintptr_t)A & 15) || ((uintptr_t)B & 15)) return false;
  if ((M / BM) * (N / BN) > 2147483647LL) return false;
  return true;
}

}  // namespace tile
}  // namespace cig
