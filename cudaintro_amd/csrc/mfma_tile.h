// The LDS-tiled MFMA GEMM kernel shared by the bf16, fp16 and int8 families.
//
// Workgroup = 256 lanes = 4 waves (2 x 2) -- or, for N x K int8 weights with a 16-bit output and
// for their 128-row tiles, 512 lanes = 8 waves (4 x 2) of half the height, two per SIMD, same data
// flow, see launch_tile_256 / launch_tile_128 --; macro tile 256 (m) x 256 (n); k is consumed in
// stages of 64 BYTES per row (32 halves, 64 int8 or 16 floats) = two MFMA k-steps.  Each wave
// owns a 128 x 128 block = 4 x 4 MFMA tiles of 32 x 32 = 256 accumulators per lane (the AGPR
// file); one wave per SIMD.  The tile height is a template parameter (MT = 4, 3, 2 or 1 row
// tiles per wave: 256, 192, 128 or 64 rows) so that small or awkward M still fill the chip; the
// text below describes MT = 4.  Both operand tiles of a stage are 16 KiB.  B stages form a
// ring of 4 slots in LDS (64 KiB), three of them in flight ahead of the one being multiplied:
// HBM/L2 latency here is of the order of a microsecond, two to three stage times.  A is
// fetched two stages at a time as whole 128-byte lines (half as many L2 requests as 64-byte
// pieces) into a ring of 3 pair slots (96 KiB): 160 KiB in all.
//
// Global -> LDS goes straight through the LDS-DMA path (global_load_lds_dwordx4): no
// staging registers, no ds_write.  One such instruction deposits the wave's 64 x 16 bytes
// contiguously in LDS, lane by lane, while each lane chooses its own global address; the
// bank-conflict swizzle is therefore applied on the global side (the chunk a lane fetches),
// and LDS slot s of a row holds chunk s ^ swizzle(row).
//
// A pair  [256 m][128 B of k] = stages 2p and 2p+1, as in memory.  16-byte chunk c of row r
//         lives at r*128 + ((c ^ ((r >> 1) & 7)) << 4): the 16-byte fragment reads of 32
//         consecutive rows then spread over all banks.
// B tile  one of
//   NK    (weights, k contiguous) row-major like A, so fetched the same way: pairs
//         [256 n][128 B of k] of whole lines, two 32 KiB pair slots in the 64 KiB of the
//         B ring, read like A (one 16-byte read per fragment: 8-byte half reads of this layout
//         would collide two ways, a wave's 32 rows falling on 16 bank groups);
//   KN16  [32 k][256 n] halves, KN8 [64 k][256 n] bytes (n contiguous, as C = A.B stores
//         B).  The MFMA wants k contiguous per lane, so fragments come from the transposing
//         LDS reads ds_read_b64_tr_b16 / _tr_b8: within 16 lanes, lane i supplies the
//         address of 8 bytes of row k0 + i/4 (i/2 for bytes) and receives the 4 (8)
//         k-values of column n0 + i.  Chunks are XOR-swizzled by k so that the rows one
//         instruction touches fall in different banks.
//
// Pipeline, iteration s (B of stage s sits in slot s % 4, A in pair slot (s / 2) % 3):
//   k-step 0: 16 MFMAs on the fragments of (s,0); under them the 12 LDS reads of (s,1)
//   wait until this wave's DMA of stage s+1 has landed (vmcnt), workgroup barrier
//   k-step 1: 16 MFMAs on (s,1); under them the 12 LDS reads of (s+1,0) and the DMA, one
//             instruction in every second MFMA slot:
//             4 instructions of B of stage s+3 into the slot stage s-1 just left (every wave
//             finished reading it before it reached the barrier) and 4 of the 8 of an A
//             pair: the first half of the pair of stages s+4, s+5 when s is even, the second
//             half of the same pair (then stages s+3, s+4) when s is odd.
// With N x K weights both operands move as pairs: even stages issue the A pair of stages s+4,
// s+5, odd stages the B pair of stages s+3, s+4 (into the slot whose last fragments were read
// in k-step 0 of that stage).
// Fragments are double buffered in registers.  The emitted order is pinned slot by slot
// with scheduling fences: one MFMA, at most one LDS read, at most one DMA.  The ring slots
// repeat every 12 stages (4 B slots, 3 A pair slots of 2 stages): the steady part of the main
// loop runs in trips of 12 stages whose slots are all compile-time constants, so that no ring
// or address arithmetic is left between the matrix instructions (see `stage` below).
//
// The MFMA is issued with the B fragment as its first operand and the A fragment as its
// second, so it yields the transposed 32 x 32 block: lane l holds, for the single output
// row m = l%32, columns 8q + 4(l/32) + e (q, e = 0..3) in accumulator 4q+e, i.e. four
// consecutive columns per quad, which the epilogue stores as one piece of a row of C.
#pragma once

#include <type_traits>

#include "common.h"
#include "tile_plan.h"

namespace cig {
namespace tile {

constexpr int OPERAND_BYTES = 256 * KB;    // 16 KiB, either operand

typedef __attribute__((address_space(3))) i16x4 lds_i16x4;
typedef __attribute__((address_space(3))) i32x2 lds_i32x2;
typedef __attribute__((address_space(3))) void lds_void;
typedef __attribute__((address_space(1))) void global_void;

// ---- A-like tile: [256 rows][4 chunks] ----------------------------------------------------
__device__ __forceinline__ int rowmajor_swz(int r) {
  return ((r >> 2) & 1) | ((((r >> 1) ^ (r >> 3)) & 1) << 1);
}
__device__ __forceinline__ int rowmajor_off(int r, int c) {
  return r * KB + ((c ^ rowmajor_swz(r)) << 4);
}

// ---- A pair tile: [64 T rows][128 B = two stages of k]: A is fetched as whole 128-byte lines,
// one pair of stages at a time (half as many L2 requests as 64-byte pieces).  Chunk c (16 B)
// of row r sits at r*128 + ((c ^ pair_swz(r)) << 4).
__device__ __forceinline__ int pair_swz(int r) { return (r >> 1) & 7; }
__device__ __forceinline__ int pair_off(int r, int c) { return r * 128 + ((c ^ pair_swz(r)) << 4); }
// one instruction = 8 rows of 128 B; wave w moves rows 16 T w .. 16 T (w + 1): 2 T instructions
template <int T>
struct RowPairDmaT {
  static __device__ __forceinline__ int dma_lds(int w, int i) { return (16 * T * w + 8 * i) * 128; }
  static __device__ __forceinline__ int64_t dma_src(int w, int i, int l, int64_t ld, int last) {
    const int r = 16 * T * w + 8 * i + (l >> 3);
    return (int64_t)(r < last ? r : last) * ld + (((l & 7) ^ pair_swz(r)) << 4);
  }
};

enum BMode { B_NK = 0, B_KN16 = 1, B_KN8 = 2, B_KN32 = 3 };

// Fragment plumbing shared by the 16-bit / int8 tiles: a B fragment is two 8-byte halves.
struct HalfPieces {
  static constexpr int NREADS = 8;  // LDS reads per k-step for the four B fragments
  typedef u32x2 piece_t;
  static __device__ __forceinline__ u32x4 bfrag(const piece_t (&b)[NREADS], int j, int) {
    return __builtin_shufflevector(b[2 * j], b[2 * j + 1], 0, 1, 2, 3);
  }
};

template <int MODE>
struct BTile;

// DMA geometry of a tile: wave w issues instruction i (0..3); the instruction fills 1 KiB of
// LDS starting at dma_lds(w, i); lane l fetches the 16 bytes at global byte offset
// dma_src(w, i, l, ld) from the tile's origin (row stride ld bytes).

// [64 T rows][64 B]: one instruction = 16 rows, wave w moves rows 16 T w .. 16 T (w + 1).
template <int T>
struct RowMajorDmaT {
  static __device__ __forceinline__ int dma_lds(int w, int i) { return (16 * T * w + 16 * i) * KB; }
  // `last` = last valid row of the tile (rows beyond it re-read it; they are never stored)
  static __device__ __forceinline__ int64_t dma_src(int w, int i, int l, int64_t ld, int last) {
    const int r = 16 * T * w + 16 * i + (l >> 2);
    return (int64_t)(r < last ? r : last) * ld + (((l & 3) ^ rowmajor_swz(r)) << 4);
  }
};
typedef RowMajorDmaT<4> RowMajorDma;

// Source of the 16-byte pieces that lie past the end of K in the last stage: the matrix
// instructions always consume whole 64-byte stages, so what K does not fill is fetched from here.
static __device__ __align__(64) uint32_t g_zero_chunk[16];

// Weights N x K: identical to the A tile.
template <>
struct BTile<B_NK> : RowMajorDma, HalfPieces {
  static __device__ __forceinline__ int dma_k(int, int, int) { return 0; }  // (fetched as pairs)
  // half h (0/1) of the fragment of column tile j, k-step kk: 8 bytes of k
  static __device__ __forceinline__ u32x2 frag_half(const char* sb, int wn, int j, int kk, int h,
                                                    int l) {
    const int r = wn * 128 + 32 * j + (l & 31);
    return *reinterpret_cast<const u32x2*>(sb + rowmajor_off(r, 2 * kk + (l >> 5)) + 8 * h);
  }
  // whole fragment (16 bytes) of column tile j from a pair tile [256 n][128 B], read like an
  // A fragment; par = which stage of the pair
  static __device__ __forceinline__ u32x4 frag_pair(const char* sb, int wn, int j, int par, int kk,
                                                    int l) {
    const int r = wn * 128 + 32 * j + (l & 31);
    return *reinterpret_cast<const u32x4*>(sb + pair_off(r, 4 * par + 2 * kk + (l >> 5)));
  }
};

// K x N halves: [32 k][32 chunks of 8 halves]; one DMA instruction = 2 k-rows.
template <>
struct BTile<B_KN16> : HalfPieces {
  static __device__ __forceinline__ int swz(int k) {
    const int k3 = k & 3;
    return (k3 << 2) | ((((k3 >> 1) ^ k3) & 1) << 1);
  }
  static __device__ __forceinline__ int off(int k, int c) { return k * 512 + ((c ^ swz(k)) << 4); }
  static __device__ __forceinline__ int dma_lds(int w, int i) { return (8 * w + 2 * i) * 512; }
  // k row (within the stage) that lane l of instruction (w, i) fetches
  static __device__ __forceinline__ int dma_k(int w, int i, int l) { return 8 * w + 2 * i + (l >> 5); }
  // `last` = last valid 16-byte chunk of a tile row (columns beyond N re-read it)
  static __device__ __forceinline__ int64_t dma_src(int w, int i, int l, int64_t ld, int last) {
    const int k = 8 * w + 2 * i + (l >> 5);
    const int c = (l & 31) ^ swz(k);
    return (int64_t)k * ld + ((c < last ? c : last) << 4);
  }
  static __device__ __forceinline__ u32x2 frag_half(const char* sb, int wn, int j, int kk, int h,
                                                    int l) {
    const int k = 16 * kk + 8 * (l >> 5) + ((l & 15) >> 2) + 4 * h;
    const int n = wn * 128 + 32 * j + 16 * ((l >> 4) & 1) + 4 * (l & 3);
    const int sub = ((n >> 2) & 1) * 8;
    i16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4*)(sb + off(k, n >> 3) + sub));
    return __builtin_bit_cast(u32x2, v);
  }
};

// K x N bytes: [64 k][16 chunks of 16 bytes]; one DMA instruction = 4 k-rows.
template <>
struct BTile<B_KN8> : HalfPieces {
  static __device__ __forceinline__ int swz(int k) {
    return ((k & 7) << 1) | (((k >> 2) ^ (k >> 4)) & 1);
  }
  static __device__ __forceinline__ int off(int k, int c) { return k * 256 + ((c ^ swz(k)) << 4); }
  static __device__ __forceinline__ int dma_lds(int w, int i) { return (16 * w + 4 * i) * 256; }
  static __device__ __forceinline__ int dma_k(int w, int i, int l) { return 16 * w + 4 * i + (l >> 4); }
  static __device__ __forceinline__ int64_t dma_src(int w, int i, int l, int64_t ld, int last) {
    const int k = 16 * w + 4 * i + (l >> 4);
    const int c = (l & 15) ^ swz(k);
    return (int64_t)k * ld + ((c < last ? c : last) << 4);
  }
  static __device__ __forceinline__ u32x2 frag_half(const char* sb, int wn, int j, int kk, int h,
                                                    int l) {
    const int k = 32 * kk + 16 * (l >> 5) + ((l & 15) >> 1) + 8 * h;
    const int n = wn * 128 + 32 * j + 16 * ((l >> 4) & 1) + 8 * (l & 1);
    const int sub = ((n >> 3) & 1) * 8;
    i32x2 v = __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_i32x2*)(sb + off(k, n >> 4) + sub));
    return __builtin_bit_cast(u32x2, v);
  }
};

// K x N fp32: [16 k][256 n] floats, rows of 1 KiB = 64 chunks; one DMA instruction = 1 k-row.
// Lane (n, g) reads the single float B[k][n] per MFMA; lanes 0-31 and 32-63 read rows k and
// k+4, which the swizzle moves 128 bytes apart.
template <>
struct BTile<B_KN32> {
  static constexpr int NREADS = 16;
  typedef uint32_t piece_t;
  static __device__ __forceinline__ int swz(int k) { return ((k >> 2) & 1) << 3; }
  static __device__ __forceinline__ int dma_lds(int w, int i) { return (4 * w + i) * 1024; }
  static __device__ __forceinline__ int dma_k(int w, int i, int) { return 4 * w + i; }
  static __device__ __forceinline__ int64_t dma_src(int w, int i, int l, int64_t ld, int last) {
    const int k = 4 * w + i;
    const int c = l ^ swz(k);
    return (int64_t)k * ld + ((c < last ? c : last) << 4);
  }
  // read idx (0..15) of k-step kk: element e = idx/4 of the fragment of column tile j = idx%4
  static __device__ __forceinline__ piece_t read(const char* sb, int wn, int idx, int kk, int l) {
    const int e = idx >> 2, j = idx & 3;
    const int k = 8 * kk + 4 * (l >> 5) + e;
    const int n = wn * 128 + 32 * j + (l & 31);
    return *reinterpret_cast<const uint32_t*>(sb + k * 1024 + (((n >> 2) ^ swz(k)) << 4) +
                                              (n & 3) * 4);
  }
  static __device__ __forceinline__ float bfrag(const piece_t (&b)[NREADS], int j, int sub) {
    return __builtin_bit_cast(float, b[4 * sub + j]);
  }
};

// read idx (0..7) of k-step kk for the half-piece tiles: half idx%2 of column tile idx/2
template <int MODE>
__device__ __forceinline__ typename BTile<MODE>::piece_t read_b_piece(const char* sb, int wn,
                                                                      int idx, int kk, int l) {
  if constexpr (MODE == B_KN32)
    return BTile<MODE>::read(sb, wn, idx, kk, l);
  else
    return BTile<MODE>::frag_half(sb, wn, idx >> 1, kk, idx & 1, l);
}

// ---- arithmetic traits ----------------------------------------------------------------------
struct MathBF16 {
  static constexpr int SUBSTEPS = 1;  // MFMAs per fragment pair
  static __device__ __forceinline__ u32x4 afrag(u32x4 a, int) { return a; }
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
  static constexpr int SUBSTEPS = 1;  // MFMAs per fragment pair
  static __device__ __forceinline__ u32x4 afrag(u32x4 a, int) { return a; }
  typedef f32x16 acc_t;
  typedef float scalar_t;
  static constexpr int ELEM_BYTES = 2;
  static __device__ __forceinline__ acc_t mfma(u32x4 first, u32x4 second, acc_t acc) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, first),
                                                  __builtin_bit_cast(f16x8, second), acc, 0, 0, 0);
  }
};
struct MathI8 {
  static constexpr int SUBSTEPS = 1;  // MFMAs per fragment pair
  static __device__ __forceinline__ u32x4 afrag(u32x4 a, int) { return a; }
  typedef i32x16 acc_t;
  typedef int32_t scalar_t;
  static constexpr int ELEM_BYTES = 1;
  static __device__ __forceinline__ acc_t mfma(u32x4 first, u32x4 second, acc_t acc) {
    return __builtin_amdgcn_mfma_i32_32x32x32_i8(__builtin_bit_cast(i32x4, first),
                                                 __builtin_bit_cast(i32x4, second), acc, 0, 0, 0);
  }
};

// fp32: v_mfma_f32_32x32x2_f32 takes one float per lane and operand (row l%32, k = l/32).
// A 16-byte fragment read gives a lane 4 consecutive k of its row, lanes 32-63 the next 4,
// so four MFMAs consume one fragment pair: MFMA e multiplies k0+e (lanes 0-31) and k0+4+e.
struct MathF32 {
  static constexpr int SUBSTEPS = 4;
  static __device__ __forceinline__ float afrag(u32x4 a, int sub) {
    const uint32_t bits = a[sub];  // (bit_cast applied directly to a vector element misreads it)
    return __builtin_bit_cast(float, bits);
  }
  typedef f32x16 acc_t;
  typedef float scalar_t;
  static constexpr int ELEM_BYTES = 4;
  static __device__ __forceinline__ acc_t mfma(float first, float second, acc_t acc) {
    return __builtin_amdgcn_mfma_f32_32x32x2f32(first, second, acc, 0, 0, 0);
  }
};

// Maps the hardware workgroup id to an output tile.  Workgroups are handed to the 8 XCDs
// round-robin; the remap gives each XCD a contiguous range of logical ids, and logical ids
// walk the tile grid in column-major groups of GROUP_M tile rows, so the tiles resident on
// one XCD at a time share A row panels and B column panels in that XCD's L2.  GROUP_M = 4
// measured best at 8192^3 (1, 2, 3, 4, 5, 6, 8, 16, 32 tried: 32 costs 35 %): the 32 resident
// tiles form 4 rows x 8 columns, each XCD keeps its own 4 A row panels for its whole share
// and all XCDs stream the same B column panels at the same time.
__device__ __forceinline__ void tile_of_workgroup(int tiles_m, int tiles_n, int& tm, int& tn) {
  constexpr int XCDS = 8, GROUP_M = 4;
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

// Split-K: the accumulators of one K range, stored raw (fp32 or int32 bits) to
// base + split * split_stride, row-major with leading dimension ld.
struct EpiNone {};
struct EpiPartialX4 {
  uint32_t* base;
  int64_t ld;
  int64_t split_stride;  // elements between the partial matrices of consecutive splits
  static constexpr int OUT_BYTES = 4;
  typedef EpiNone row_t;
  typedef EpiNone col_t;
  __device__ __forceinline__ row_t load_row(int64_t) const { return row_t{}; }
  __device__ __forceinline__ col_t load_cols(int64_t) const { return col_t{}; }
  template <typename T>
  __device__ __forceinline__ u32x4 pack(row_t, col_t, T v0, T v1, T v2, T v3) const {
    return u32x4{__builtin_bit_cast(uint32_t, v0), __builtin_bit_cast(uint32_t, v1),
                 __builtin_bit_cast(uint32_t, v2), __builtin_bit_cast(uint32_t, v3)};
  }
  template <typename T>
  __device__ __forceinline__ u32x4 pack(int64_t, int64_t, T v0, T v1, T v2, T v3) const {
    return pack(row_t{}, col_t{}, v0, v1, v2, v3);
  }
  __device__ __forceinline__ char* out_row(int64_t r) const {
    return reinterpret_cast<char*>(base + r * ld);
  }
  template <typename T>
  __device__ __forceinline__ void side(int64_t, int64_t, T, T, T, T) const {}
  EpiPartialX4 shift_cols(int64_t c0) const { return EpiPartialX4{base + c0, ld, split_stride}; }
};
// An epilogue may declare `static constexpr bool HAS_UNIFORM_MODE = true` (see epilogues.h).
template <typename E, typename = void>
struct epi_has_uniform_mode : std::false_type {};
template <typename E>
struct epi_has_uniform_mode<E, typename std::enable_if<E::HAS_UNIFORM_MODE>::type>
    : std::true_type {};

// Measurement aid: an epilogue that declares `static constexpr bool PROFILED = true` and carries
// `uint64_t* stamps` makes the kernel record, per workgroup, the shader-clock counter and the
// constant-rate counter at four points: start, first stage landed, main loop done, epilogue done
// (stamps[8 * workgroup + 2 * point + {0, 1}]; at the first point the hardware id of the unit
// the workgroup runs on takes the place of the shader-clock count).
template <typename E, typename = void>
struct epi_profiled : std::false_type {};
template <typename E>
struct epi_profiled<E, typename std::enable_if<E::PROFILED>::type> : std::true_type {};
template <typename Epi>
struct EpiProfiled : Epi {
  uint64_t* stamps;
  // Non-zero: every workgroup computes output tile (0, 0) instead of its own (all of them read
  // the same two operand panels, which then stay in every L2, and store the same values to the
  // same place): what the launch would take if no operand read ever left the L2.
  int same_tile;
  static constexpr bool PROFILED = true;
};

// The epilogue of K range `split` (blockIdx.y): only the partial store depends on it.
template <typename Epi>
__device__ __forceinline__ Epi epilogue_of_split(const Epi& e, int) { return e; }
__device__ __forceinline__ EpiPartialX4 epilogue_of_split(const EpiPartialX4& e, int split) {
  return EpiPartialX4{e.base + split * e.split_stride, e.ld, e.split_stride};
}

// The epilogue of the tile kernels: accumulators -> output rows.
// acc[i][j][4q+e] = C[m0 + wm*32*MT + 32i + l%32][n0 + wn*128 + 32j + 8q + 4g + e]: a lane
// holds short pieces of 32 different rows.  Each wave stages one 32-row x 128-column block
// at a time in its own piece of the (now idle) LDS and writes it out as whole rows: every
// store instruction then covers full 256- or 512-byte row segments.  Call it once every wave
// of the workgroup has stopped reading the operand ring and no DMA is in flight.
template <typename Math, int MT, int NW, int TILE_M, typename Epi>
__device__ __forceinline__ void store_tile(const Epi& epi, typename Math::acc_t (&acc)[MT][4],
                                           char* lds, int w, int wm, int wn, int64_t m0,
                                           int64_t n0, int M, int N, float epi_row_word,
                                           float epi_col_word) {
  // The epilogue takes the lane number afresh from the hardware (and opaque to the compiler),
  // so that neither it nor any of the epilogue's addresses is held in a register through the
  // main loop.
  int le = __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
  asm volatile("" : "+v"(le));
  le &= 63;
  const int ge = le >> 5;
  constexpr int OB = Epi::OUT_BYTES;
  constexpr int ROW_BYTES = 128 * OB;
  constexpr int ROW_STRIDE = ROW_BYTES + 16;
  constexpr int LANES_PER_ROW = ROW_BYTES / 16;
  constexpr int ROWS_PER_PASS = 64 / LANES_PER_ROW;
  // (the launcher sizes the dynamic LDS for the larger of the ring and these staging blocks)
  static_assert(NW * 32 * ROW_STRIDE <= 160 * 1024, "the waves' staging blocks must fit the LDS");
  char* scr = lds + w * (32 * ROW_STRIDE);
  typedef decltype(epi.pack((int64_t)0, (int64_t)0, acc[0][0][0], acc[0][0][0], acc[0][0][0],
                            acc[0][0][0])) packed_t;
  // What the epilogue needs per column quad (scales, bias) is the same for every row tile:
  // fetched once, up front, so that no load latency sits between the accumulator reads.
  typename Epi::col_t colv[4][4];
  bool cols_done = false;
  if constexpr (epi_has_uniform_mode<Epi>::value) {
    if (epi.col_uniform()) {
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int q = 0; q < 4; ++q) colv[j][q] = epi.cols_from_word(epi_col_word);
      cols_done = true;
    }
  }
  if (!cols_done) {
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int64_t col = n0 + wn * 128 + 32 * j + 8 * q + 4 * ge;
        colv[j][q] = epi.load_cols(col < N ? col : N - 4);
      }
  }
  // Store side of the staging: lane -> (row within a pass, 16-byte piece of the 128-column row).
  // N is a multiple of 4: a piece of 32-bit outputs is in or out as a whole, one of 16-bit
  // outputs may be half inside (then its first 8 bytes are stored).
  constexpr int NPASS = 32 / ROWS_PER_PASS;
  const int lane_row = le / LANES_PER_ROW, c16 = le % LANES_PER_ROW;
  const int64_t piece_col = n0 + wn * 128 + c16 * (16 / OB);
  const bool piece_in = piece_col < N;
  const bool piece_half = OB == 2 && piece_col + 8 > N;
  const int64_t row_step = (intptr_t)epi.out_row(1) - (intptr_t)epi.out_row(0);  // bytes per row
  const bool interior = m0 + TILE_M <= M && n0 + BN <= N;  // (uniform)
#pragma unroll
  for (int i = 0; i < MT; ++i) {
    const int64_t row0 = m0 + wm * 32 * MT + 32 * i;
    const int64_t row = row0 + (le & 31);
    const bool row_ok = row < M;
    const int64_t row_c = row_ok ? row : M - 1;  // scale lookups stay in bounds
    typename Epi::row_t rowv;
    if constexpr (epi_has_uniform_mode<Epi>::value)
      rowv = epi.row_uniform() ? epi.row_from_word(epi_row_word) : epi.load_row(row_c);
    else
      rowv = epi.load_row(row_c);
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int c = 32 * j + 8 * q + 4 * ge;
        const int64_t col = n0 + wn * 128 + c;
        const bool col_ok = col < N;  // N is a multiple of 4: a quad is in or out as a whole
        *reinterpret_cast<packed_t*>(scr + (le & 31) * ROW_STRIDE + c * OB) =
            epi.pack(rowv, colv[j][q], acc[i][j][4 * q + 0], acc[i][j][4 * q + 1],
                     acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]);
        if (row_ok && col_ok)
          epi.side(row, col, acc[i][j][4 * q + 0], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2],
                   acc[i][j][4 * q + 3]);
      }
    // All pieces of the block are read back into registers first and then stored: one LDS
    // latency per row tile instead of one per store instruction.  Row addresses advance by a
    // constant; the bounds checks exist only in workgroups on the matrix edge.
    u32x4 v[NPASS];
#pragma unroll
    for (int p = 0; p < NPASS; ++p)
      v[p] = *reinterpret_cast<const u32x4*>(scr + (p * ROWS_PER_PASS + lane_row) * ROW_STRIDE +
                                             c16 * 16);
    __builtin_amdgcn_sched_barrier(0);
    char* dst0 = epi.out_row(row0 + lane_row) + (n0 + wn * 128) * OB + c16 * 16;
    if (interior) {
#pragma unroll
      for (int p = 0; p < NPASS; ++p)
        // streaming stores: C is not read again by this kernel and should not evict A / B
        __builtin_nontemporal_store(v[p],
                                    reinterpret_cast<u32x4*>(dst0 + p * ROWS_PER_PASS * row_step));
    } else {
#pragma unroll
      for (int p = 0; p < NPASS; ++p) {
        char* dst = dst0 + p * ROWS_PER_PASS * row_step;
        if (row0 + p * ROWS_PER_PASS + lane_row < M && piece_in) {
          if (piece_half)
            __builtin_nontemporal_store(u32x2{v[p][0], v[p][1]}, reinterpret_cast<u32x2*>(dst));
          else
            __builtin_nontemporal_store(v[p], reinterpret_cast<u32x4*>(dst));
        }
      }
    }
  }
}

// Epi: an epilogue functor (see epilogues.h): load_row / load_cols / pack / side / out_row.
//
// A, B are byte pointers; lda/ldb are in BYTES.  Any M; N a multiple of 4; all rows 16-byte
// aligned (tile_shape_ok checks).  grid = (tiles, K ranges): range y covers the bytes
// [y * k_range_bytes, min((y + 1) * k_range_bytes, k_total_bytes)) of k; k_range_bytes is a
// whole number of 64-byte stages whenever there is more than one range, so only the last
// range can be shorter than the others or leave its last stage partly filled (the pieces
// past its end are fetched as zeros).  k_total_bytes is a multiple of 16.
template <typename Math, int BMODE, int NSTAGES, int MT, typename Epi, int WM = 2>
__global__ __launch_bounds__(128 * WM, 1) void mfma_tile_kernel(int M, int N, int tiles_m,
                                                           int tiles_n, int k_range_bytes,
                                                           int k_total_bytes,
                                                           const char* __restrict__ A,
                                                           int64_t lda,
                                                           const char* __restrict__ B,
                                                           int64_t ldb, Epi epi_all,
                                                           int64_t a_split_step,
                                                           int64_t b_split_step) {
  // blockIdx.y = K range (split-K launches only): each starts a_split_step / b_split_step
  // bytes after the one before; k_bytes = bytes of k in this one, KTS = its stages
  const int k_left = k_total_bytes - (int)blockIdx.y * k_range_bytes;
  const int k_bytes = k_left < k_range_bytes ? k_left : k_range_bytes;
  const int KTS = (k_bytes + KB - 1) / KB;
  const Epi epi = epilogue_of_split(epi_all, (int)blockIdx.y);
  A += blockIdx.y * a_split_step;
  B += blockIdx.y * b_split_step;
  typedef typename Math::acc_t acc_t;
  typedef BTile<BMODE> BT;
  constexpr int DIST = NSTAGES - 1;  // stages in flight ahead of the one being multiplied
  constexpr int NW = 2 * WM;             // waves: WM rows of 2
  constexpr int TILE_M = 32 * MT * WM;   // rows of the macro tile
  static_assert(NSTAGES == 4, "the wait counts below assume three stages in flight");
  // N x K weights are row-major like A: they too are fetched as whole 128-byte lines, a pair
  // of stages at a time, into two 32 KiB pair slots (the same 64 KiB as the ring of four
  // single stages the K x N layouts use).
  constexpr bool BPAIR = BMODE == B_NK;
  constexpr int DMA_A = TILE_M / 8 / NW;        // per wave and stage pair: A instructions of 1 KiB
  // per wave: B instructions per stage pair (N x K weights) / per stage
  constexpr int DMA_B = (BPAIR ? 32 : 16) / NW;
  constexpr int BPAIR_BYTES = 256 * 128;
  constexpr int APAIR_BYTES = TILE_M * 128;
  constexpr int B_RING = NSTAGES * OPERAND_BYTES;   // B slots first, then three A pair slots
  typedef RowPairDmaT<1> PairDma;   // instruction q = rows 8 q .. 8 q + 7: (q >> 1, q & 1)
  extern __shared__ __attribute__((aligned(1024))) char lds[];
  const int t = threadIdx.x;
  const int l = t & 63;
  const int w = __builtin_amdgcn_readfirstlane(t >> 6);
  const int wm = w >> 1, wn = w & 1;
  auto stamp = [&](int point) {
    if constexpr (epi_profiled<Epi>::value) {
      if (threadIdx.x == 0) {
        uint64_t* p = epi.stamps + ((int64_t)blockIdx.y * gridDim.x + blockIdx.x) * 8 + 2 * point;
        // (point 0 carries, in place of the shader-clock count nobody reads there, where the
        // workgroup runs: HW_ID in the low word, XCC_ID above it)
        p[0] = point == 0 ? ((uint64_t)__builtin_amdgcn_s_getreg((3 << 11) | 20) << 32) |
                                __builtin_amdgcn_s_getreg((31 << 11) | 4)
                          : __builtin_amdgcn_s_memtime();
        p[1] = __builtin_amdgcn_s_memrealtime();
      }
    }
  };
  stamp(0);

  int tm, tn;
  tile_of_workgroup(tiles_m, tiles_n, tm, tn);
  // (the divisions above run on the vector unit: tell the compiler the results are uniform,
  // so that everything derived from them, the DMA base addresses above all, stays scalar)
  tm = __builtin_amdgcn_readfirstlane(tm);
  tn = __builtin_amdgcn_readfirstlane(tn);
  if constexpr (epi_profiled<Epi>::value) {
    if (epi.same_tile) tm = tn = 0;
  }
  const int64_t m0 = (int64_t)tm * TILE_M, n0 = (int64_t)tn * BN;
  // Per-tensor operands of the epilogue: one word each at a uniform address, read here, before
  // anything is written, hence with a scalar load whose latency nothing waits for.
  float epi_row_word = 0.0f, epi_col_word = 0.0f;
  if constexpr (epi_has_uniform_mode<Epi>::value) {
    epi_row_word = *epi.row_word();
    epi_col_word = *epi.col_word();
  }

  // ---- DMA sources: uniform tile origin + per-lane byte offsets ------------------------------
  const char* a_tile = A + m0 * lda;  // + stage * KB
  const char* b_tile;                 // + stage * b_kstep
  int64_t b_kstep;
  if (BMODE == B_NK) {
    b_tile = B + n0 * ldb;
    b_kstep = KB;
  } else {
    b_tile = B + n0 * Math::ELEM_BYTES;
    b_kstep = (int64_t)(KB / Math::ELEM_BYTES) * ldb;
  }
  // Ragged edges: rows past M (and, for N x K weights, past N) re-read the last valid row,
  // column chunks past N (K x N operands) re-read the last valid chunk; what they produce
  // is never stored.
  const int a_last = (int)((M - 1 - m0) < (TILE_M - 1) ? (M - 1 - m0) : (TILE_M - 1));
  const int n_left = (int)((N - n0) < BN ? (N - n0) : BN);
  const int b_last = BMODE == B_NK ? n_left - 1 : (n_left * Math::ELEM_BYTES + 15) / 16 - 1;
  // The last pair of stages may be filled only in part (an odd number of stages, or a K that
  // does not fill its last stage): pair_valid = 16-byte pieces of it that lie inside this K
  // range (1..8), tail_k = bytes of k inside the last stage (16..64).  What lies beyond is
  // fetched from a block of zeros instead (reading on would leave the row, and for the last
  // rows the matrix), so the matrix instructions see zero operands there.
  const int last_pair = (KTS - 1) >> 1;
  const int pair_valid = (k_bytes - last_pair * 128) >> 4;
  const int tail_k = k_bytes - (KTS - 1) * KB;
  const char* const zero_src = reinterpret_cast<const char*>(g_zero_chunk);
  uint32_t a_voff[DMA_A], b_voff[DMA_B];
#pragma unroll
  for (int i = 0; i < DMA_A; ++i) {
    const int q = DMA_A * w + i;
    a_voff[i] = (uint32_t)PairDma::dma_src(q >> 1, q & 1, l, lda, a_last);
  }
#pragma unroll
  for (int i = 0; i < DMA_B; ++i) {
    const int q = DMA_B * w + i;
    b_voff[i] = BPAIR ? (uint32_t)PairDma::dma_src(q >> 1, q & 1, l, ldb, b_last)
                      : (uint32_t)BT::dma_src(q >> 2, q & 3, l, ldb, b_last);
  }

  // The DMA instructions are written as asm so that the compiler's wait-count insertion does
  // not know them: it would otherwise make every later LDS read it cannot tell apart (the
  // transposing reads) wait for all outstanding DMA.  Completion is waited for by hand
  // (vmcnt) before the barrier that publishes a stage.  M0 carries the wave-uniform LDS
  // destination; lane l's 16 bytes land at M0 + 16 l.  The source is a scalar base (tile origin
  // + stage, advanced on the scalar unit) plus a loop-invariant 32-bit lane offset: no vector
  // ALU work per instruction (on this chip every vector instruction between two matrix
  // instructions delays the second, by about a cycle under the 16-bit and int8 ones and by
  // ten and more under the fp32 one, which runs on the vector ALU's own multipliers).
  const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)lds;
  auto dma16 = [&](const char* base, uint32_t voff, uint32_t lds_dst) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :
                 : "s"(lds_dst), "v"(voff), "s"(base)
                 : "m0");
  };
  // the same with a full per-lane address: lanes with `zero` set fetch zeros
  auto dma16z = [&](const char* base, uint32_t voff, uint32_t lds_dst, bool zero) {
    const char* src = zero ? zero_src : base + voff;
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off"
                 :
                 : "s"(lds_dst), "v"(src)
                 : "m0");
  };
  // piece (16 bytes of k) that lane l fetches with pair instruction q (rows 8 q .. 8 q + 7)
  auto pair_piece = [&](int q) { return (l & 7) ^ ((4 * (q & 1) + (l >> 4)) & 7); };
  // d < DMA_B: B instruction d of stage `st` (of its stage pair, for N x K weights) into B
  // slot `slot`; above: A instruction d - DMA_B of the stage pair st / 2 into pair slot `pslot`.
  // Past the last stage the last one is fetched
  // again (into slots nobody reads any more), which keeps the number of outstanding
  // instructions, and so the vmcnt waits, uniform.
  // `steady_const`: the caller guarantees st < KTS and a pair that is not the odd tail, so
  // that no per-lane arithmetic is left: the uniform part of the address is a scalar base.
  auto dma_piece = [&](int st, int slot, int pslot, int d, auto steady_const) {
    constexpr bool STEADY = decltype(steady_const)::value;
    if (!STEADY) st = st < KTS ? st : KTS - 1;
    // (no branches here: the instruction order of a stage is pinned slot by slot)
    const bool last_pair_now = !STEADY && (st >> 1) == last_pair;
    if (d < DMA_B) {
      const int q = DMA_B * w + d;
      if (BPAIR) {
        const uint32_t dst = lds_base + slot * BPAIR_BYTES + PairDma::dma_lds(q >> 1, q & 1);
        if (STEADY)
          dma16(b_tile + (int64_t)(st >> 1) * 128, b_voff[d], dst);
        else
          dma16z(b_tile + (int64_t)(st >> 1) * 128, b_voff[d], dst,
                 last_pair_now && pair_piece(q) >= pair_valid);
      } else {
        const uint32_t dst = lds_base + slot * OPERAND_BYTES + BT::dma_lds(q >> 2, q & 3);
        if (STEADY)
          dma16(b_tile + (int64_t)st * b_kstep, b_voff[d], dst);
        else
          dma16z(b_tile + (int64_t)st * b_kstep, b_voff[d], dst,
                 st == KTS - 1 && BT::dma_k(q >> 2, q & 3, l) * Math::ELEM_BYTES >= tail_k);
      }
    } else {
      const int q = DMA_A * w + d - DMA_B;
      const uint32_t dst = lds_base + B_RING + pslot * APAIR_BYTES + PairDma::dma_lds(q >> 1, q & 1);
      if (STEADY)
        dma16(a_tile + (int64_t)(st >> 1) * 128, a_voff[d - DMA_B], dst);
      else
        dma16z(a_tile + (int64_t)(st >> 1) * 128, a_voff[d - DMA_B], dst,
               last_pair_now && pair_piece(q) >= pair_valid);
    }
  };
  typedef std::integral_constant<bool, true> steady_t;
  typedef std::integral_constant<bool, false> drain_t;

  const int a_frag_row = wm * 32 * MT + (l & 31);
  const int g = l >> 5;

  // One k-step's operands: MT A fragments (16 B each) and the pieces of the 4 B fragments.
  // N x K pairs: one 16-byte read per B fragment, kept behind the A fragments in Frags::a
  constexpr int NREAD_B = BPAIR ? 4 : BT::NREADS;
  constexpr int NREAD = MT + NREAD_B;                  // LDS reads per k-step
  constexpr int NMFMA = 4 * MT * Math::SUBSTEPS;       // MFMAs per k-step
  constexpr int READS_PER_SLOT = (NREAD + NMFMA - 1) / NMFMA;
  static_assert(DMA_A % 2 == 0, "an A pair is issued in two halves");
  // DMA instruction d of the NDMA a k-step issues goes into MFMA slot d * NMFMA / NDMA: spread
  // evenly over the k-step.  The four waves leave the barrier together, and a compute unit's one
  // address path takes about 16 cycles per 1 KiB instruction: issued back to back, one per
  // 32-cycle matrix instruction from every wave, they queue up and stall the waves' issue (a
  // register-resident loop with the stage's 8 instructions in its first 8 slots after a barrier
  // takes 1130 cycles per stage, in every second slot 1033, without any 1029).
  // (first and one-past-last DMA instruction of slot sl)
  constexpr auto dma_begin_of_slot = [](int sl, int ndma) constexpr {
    return ndma <= NMFMA ? (sl * ndma + NMFMA - 1) / NMFMA : sl * ((ndma + NMFMA - 1) / NMFMA);
  };
  struct Frags {
    u32x4 a[BPAIR ? MT + 4 : MT];
    typename BT::piece_t b[BPAIR ? 1 : BT::NREADS];
  };
  // LDS read r of k-step kk of the stage in ring slot `slot`: first the A fragments, then B.
  // `par` = parity of the stage: which half of the pair's 128-byte rows.
  auto read_piece = [&](Frags& f, int slot, int pslot, int par, int kk, int r) {
    if (r < MT)
      f.a[r] = *reinterpret_cast<const u32x4*>(
          lds + B_RING + pslot * APAIR_BYTES + pair_off(a_frag_row + 32 * r, 4 * par + 2 * kk + g));
    else if constexpr (BPAIR) {
      f.a[r] = BT::frag_pair(lds + slot * BPAIR_BYTES, wn, r - MT, par, kk, l);
    } else {
      f.b[r - MT] = read_b_piece<BMODE>(lds + slot * OPERAND_BYTES, wn, r - MT, kk, l);
    }
  };

  acc_t acc[MT][4];
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0;

  // MFMA m of a k-step: sub-step outermost, then column tile j, then row tile i: the first
  // MT need all A fragments (the first reads) but only the first pieces of B.  The row tiles
  // run up for even j and down for odd j, so that every MFMA shares one source operand with
  // the one before it (measured: 0.3-0.6 % less time at 8192^3 with one wave per SIMD).
  auto mfma_piece = [&](const Frags& f, int m) {
    const int sub = m / (4 * MT), j = (m % (4 * MT)) / MT;
    const int i = (j & 1) ? MT - 1 - m % MT : m % MT;
    if constexpr (BPAIR)
      acc[i][j] = Math::mfma(f.a[MT + j], Math::afrag(f.a[i], sub), acc[i][j]);
    else
      acc[i][j] = Math::mfma(BT::bfrag(f.b, j, sub), Math::afrag(f.a[i], sub), acc[i][j]);
  };

  Frags f0, f1;

  // s_waitcnt vmcnt(n), everything else unconstrained: vmcnt is split over bits 3:0 and 15:14.
  auto wait_vmcnt = [](auto n_const) {
    constexpr int n = decltype(n_const)::value;
    __builtin_amdgcn_s_waitcnt(0x0f70 | (n & 15) | ((n >> 4) << 14));
  };

  // prologue, in the order the main loop keeps -- single B stages: B[0], A pair 0, B[1], B[2],
  // A pair 1; B pairs: B pair 0, A pair 0, B pair 1, A pair 1 -- then stage 0 landed and the
  // first fragments in registers
#pragma unroll
  for (int d = 0; d < DMA_B + DMA_A; ++d) dma_piece(0, 0, 0, d, drain_t{});
  if (!BPAIR) {
#pragma unroll
    for (int d = 0; d < DMA_B; ++d) dma_piece(1, 1, 0, d, drain_t{});
  }
#pragma unroll
  for (int d = 0; d < DMA_B + DMA_A; ++d) dma_piece(2, BPAIR ? 1 : 2, 1, d, drain_t{});
  wait_vmcnt(std::integral_constant<int, BPAIR ? DMA_B + DMA_A : 2 * DMA_B + DMA_A>{});
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int r = 0; r < NREAD; ++r) read_piece(f0, 0, 0, 0, 0, r);
  stamp(1);
  // Single B stages: ring slots of the stage being multiplied, of the next one, and of the one
  // the DMA fills (wave-uniform scalars, advanced modulo NSTAGES each stage).  B pairs: the
  // slot of the pair being multiplied and the other one, swapped every second stage; the DMA
  // refills the current one once its last fragments are in registers.  The three A pair slots
  // advance every second stage.
  int slot = 0, next_slot = 1, dma_slot = DIST;
  int pslot = 0, next_pslot = 1, dma_pslot = 2;
  // One stage; PAR = its parity.  Single B stages: every stage issues B[s+3] and half of an A
  // pair: an even stage the first half of the pair of stages s+4, s+5 (its slot, one of three,
  // has been free since the stage before), the odd stage after it the second half.  B pairs:
  // even stages issue the A pair of stages s+4, s+5 (same slot rule), odd stages the B pair
  // of stages s+3, s+4 (its slot, one of two, is the one this stage stops reading): the
  // instructions of a stage pair are spread over both of its stages.
  // PHASE = s mod 12 when the caller knows it (the rings have periods of 4 and 6 stages), else
  // -1.  With a known phase every ring slot of the stage is a constant: the LDS addresses of its
  // fragment reads become a loop-invariant lane offset plus an immediate, the DMA destinations
  // immediates too, and the stage carries no ring arithmetic at all.  With one wave per SIMD
  // every instruction costs that wave four issue cycles, and only about seven fit under one
  // matrix instruction: the 12-stage body takes 1060 cycles per stage where the one that
  // computes its slots takes 1200.
  auto stage = [&](int s, auto par_const, auto steady_const, auto phase_const) {
    constexpr int PAR = decltype(par_const)::value;
    constexpr int PHASE = decltype(phase_const)::value;
    static_assert(PHASE < 0 || (PHASE & 1) == PAR, "the phase fixes the parity");
    constexpr int NDMA = BPAIR ? (PAR ? DMA_B : DMA_A) : DMA_B + DMA_A / 2;
    int slot_c = slot, next_slot_c = next_slot, dma_slot_c = dma_slot;
    int pslot_c = pslot, next_pslot_c = next_pslot, dma_pslot_c = dma_pslot;
    if constexpr (PHASE >= 0) {
      slot_c = BPAIR ? (PHASE / 2) % 2 : PHASE % NSTAGES;
      next_slot_c = BPAIR ? 1 - slot_c : (PHASE + 1) % NSTAGES;
      dma_slot_c = (PHASE + DIST) % NSTAGES;
      pslot_c = (PHASE / 2) % 3;
      next_pslot_c = (PHASE / 2 + 1) % 3;
      dma_pslot_c = (PHASE / 2 + 2) % 3;
    }
#pragma unroll
    for (int sl = 0; sl < NMFMA; ++sl) {
      mfma_piece(f0, sl);
#pragma unroll
      for (int r = sl * READS_PER_SLOT; r < (sl + 1) * READS_PER_SLOT; ++r)
        if (r < NREAD) read_piece(f1, slot_c, pslot_c, PAR, 1, r);
      __builtin_amdgcn_sched_barrier(0);
    }
    if (BPAIR) {
      // Odd stage: the next pair of both operands landed (only the A pair issued one stage ago
      // may still be in flight); this wave's last reads of the current B pair slot are
      // complete before any wave refills it after the barrier.  Even stage: stage s+1 is in
      // the pair already landed.
      if (PAR) {
        wait_vmcnt(std::integral_constant<int, DMA_A>{});
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      }
    } else {
      // stage s+1 landed for this wave.  Still in flight, in issue order after what stage
      // s+1 needs: even s: the first half of the A pair (s+2, s+3), B[s+2] and its second
      // half; odd s: B[s+2] and the first half of the A pair (s+3, s+4).
      wait_vmcnt(std::integral_constant<int, PAR ? DMA_B + DMA_A / 2 : DMA_B + DMA_A>{});
    }
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int sl = 0; sl < NMFMA; ++sl) {
      mfma_piece(f1, sl);
#pragma unroll
      for (int r = sl * READS_PER_SLOT; r < (sl + 1) * READS_PER_SLOT; ++r)
        if (r < NREAD)
          read_piece(f0, BPAIR ? (PAR ? next_slot_c : slot_c) : next_slot_c, PAR ? next_pslot_c : pslot_c,
                     PAR ^ 1, 0, r);
#pragma unroll
      for (int dd = 0; dd < (NDMA + NMFMA - 1) / NMFMA; ++dd) {  // (a constant trip count)
        const int d = dma_begin_of_slot(sl, NDMA) + dd;
        if (d < dma_begin_of_slot(sl + 1, NDMA) && d < NDMA) {
          if (BPAIR) {
            if (PAR)
              dma_piece(s + DIST, slot_c, dma_pslot_c, d, steady_const);           // B pair
            else
              dma_piece(s + DIST + 1, slot_c, dma_pslot_c, DMA_B + d, steady_const);  // A pair
          } else if (d < DMA_B) {
            dma_piece(s + DIST, dma_slot_c, dma_pslot_c, d, steady_const);         // B[s+3]
          } else {
            // half of the A pair the DMA is filling: stages s+4, s+5 seen from an even stage,
            // s+3, s+4 from the odd stage after it
            dma_piece(PAR ? s + DIST : s + DIST + 1, dma_slot_c, dma_pslot_c,
                      d + (PAR ? DMA_A / 2 : 0), steady_const);
          }
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    if constexpr (PHASE < 0) {
      if (BPAIR) {
        if (PAR) {
          const int tmp = slot;
          slot = next_slot;
          next_slot = tmp;
        }
      } else {
        slot = next_slot;
        next_slot = next_slot + 1 == NSTAGES ? 0 : next_slot + 1;
        dma_slot = dma_slot + 1 == NSTAGES ? 0 : dma_slot + 1;
      }
      if (PAR) {
        pslot = next_pslot;
        next_pslot = next_pslot + 1 == 3 ? 0 : next_pslot + 1;
        dma_pslot = dma_pslot + 1 == 3 ? 0 : dma_pslot + 1;
      }
    }
  };
  // Steady part: every stage the DMA reaches (up to s + 5) exists and its pair is whole.
  const int steady_end = (pair_valid < 8 && !(KTS & 1)) ? KTS - 2 : KTS;
  typedef std::integral_constant<int, -1> any_phase_t;
  int s = 0;
  // The steady part, in stage pairs (s, s + 1) with s + 5 < steady_end, every ring slot a
  // constant: whole trips of twelve stages, then up to five more pairs as straight-line code
  // whose phases go on from 0 (s is a multiple of 12 there).  The slot variables are not kept up
  // to date meanwhile.
#define CIG_STEADY_PAIR(P)                                                                      \
  stage(s, std::integral_constant<int, 0>{}, steady_t{}, std::integral_constant<int, P>{});     \
  stage(s + 1, std::integral_constant<int, 1>{}, steady_t{}, std::integral_constant<int, P + 1>{}); \
  s += 2;
  const int steady_pairs = steady_end > 5 ? (steady_end - 4) / 2 : 0;
  const int rest_pairs = steady_pairs % 6;
  for (int trip = steady_pairs / 6; trip > 0; --trip) {
    CIG_STEADY_PAIR(0)
    CIG_STEADY_PAIR(2)
    CIG_STEADY_PAIR(4)
    CIG_STEADY_PAIR(6)
    CIG_STEADY_PAIR(8)
    CIG_STEADY_PAIR(10)
  }
  if (rest_pairs > 0) {
    CIG_STEADY_PAIR(0)
    if (rest_pairs > 1) {
      CIG_STEADY_PAIR(2)
      if (rest_pairs > 2) {
        CIG_STEADY_PAIR(4)
        if (rest_pairs > 3) {
          CIG_STEADY_PAIR(6)
          if (rest_pairs > 4) {
            CIG_STEADY_PAIR(8)
          }
        }
      }
    }
  }
#undef CIG_STEADY_PAIR
  // ... then the drain, whose stages advance the slots at run time, from the slots of stage s
  slot = BPAIR ? (s / 2) % 2 : s % NSTAGES;
  next_slot = BPAIR ? 1 - slot : (s + 1) % NSTAGES;
  dma_slot = (s + DIST) % NSTAGES;
  pslot = (s / 2) % 3;
  next_pslot = (s / 2 + 1) % 3;
  dma_pslot = (s / 2 + 2) % 3;
  for (; s + 1 < KTS; s += 2) {
    stage(s, std::integral_constant<int, 0>{}, drain_t{}, any_phase_t{});
    stage(s + 1, std::integral_constant<int, 1>{}, drain_t{}, any_phase_t{});
  }
  // odd stage count: the last one
  if (KTS & 1) stage(KTS - 1, std::integral_constant<int, 0>{}, drain_t{}, any_phase_t{});
  wait_vmcnt(std::integral_constant<int, 0>{});  // no DMA outlives the main loop
  __syncthreads();  // ... for any wave, and every wave is done reading the ring
  stamp(2);

  // ---- epilogue -----------------------------------------------------------------------------
  store_tile<Math, MT, NW, TILE_M>(epi, acc, lds, w, wm, wn, m0, n0, M, N, epi_row_word,
                                   epi_col_word);
  if constexpr (epi_profiled<Epi>::value) {
    // the epilogue ends when this wave's stores have been acknowledged
    wait_vmcnt(std::integral_constant<int, 0>{});
    stamp(3);
  }
}

constexpr int DEFAULT_STAGES = 4;

// `splits` must be a value k_ranges() returned for this K (1 = the whole of K in one range).
template <typename Math, int BMODE, int MT, typename Epi, int WM = 2>
void launch_tile_mt(cigemmContext* ctx, int64_t M, int64_t N, int64_t K_bytes, const void* A,
                    int64_t lda_bytes, const void* B, int64_t ldb_bytes, const Epi& epi,
                    int splits = 1) {
  constexpr int NSTAGES = DEFAULT_STAGES;
  constexpr int TILE_M = 32 * MT * WM;
  constexpr int RING_BYTES = NSTAGES * OPERAND_BYTES + 3 * (TILE_M * 128);
  constexpr int STAGING_BYTES = 2 * WM * 32 * (128 * Epi::OUT_BYTES + 16);   // epilogue, per wave
  constexpr int LDS_BYTES = RING_BYTES > STAGING_BYTES ? RING_BYTES : STAGING_BYTES;
  auto kern = mfma_tile_kernel<Math, BMODE, NSTAGES, MT, Epi, WM>;
  static std::atomic<uint64_t> lds_set{0};  // one per template instance
  if (!ensure_dynamic_lds(ctx, (const void*)kern, LDS_BYTES, lds_set)) return;
  const int tiles_m = (int)((M + TILE_M - 1) / TILE_M), tiles_n = (int)((N + BN - 1) / BN);
  int64_t range_stages = 0;
  splits = k_ranges(K_bytes, splits, &range_stages);
  ctx->last_tile_rows = TILE_M;
  ctx->last_k_splits = splits;
  ctx->last_waves = 2 * WM;
  ctx->last_per_cu = 1;
  const int64_t range_bytes = splits > 1 ? range_stages * KB : K_bytes;
  const int64_t a_step = range_stages * KB;
  const int64_t b_step =
      BMODE == B_NK ? range_stages * KB : range_stages * (KB / Math::ELEM_BYTES) * ldb_bytes;
  hipLaunchKernelGGL(kern, dim3((unsigned)(tiles_m * tiles_n), (unsigned)splits), dim3(128 * WM),
                     LDS_BYTES, ctx->stream, (int)M, (int)N, tiles_m, tiles_n, (int)range_bytes,
                     (int)K_bytes, static_cast<const char*>(A), lda_bytes,
                     static_cast<const char*>(B), ldb_bytes, epi, a_step, b_step);
}

// Second half of a split-K GEMM: sums the `splits` partial matrices in split order (the
// result does not depend on timing) and applies the real epilogue, four columns per lane.
template <typename Scalar, typename Epi>
__global__ __launch_bounds__(256) void splitk_reduce_kernel(int M, int N, int splits,
                                                            const uint32_t* __restrict__ part,
                                                            int64_t split_stride, Epi epi) {
  const int64_t quads_per_row = N / 4, quads = (int64_t)M * quads_per_row;
  for (int64_t q = (int64_t)blockIdx.x * 256 + threadIdx.x; q < quads;
       q += (int64_t)gridDim.x * 256) {
    const int64_t r = q / quads_per_row, c = (q % quads_per_row) * 4;
    const uint32_t* p = part + r * N + c;
    // (element-wise: a bit cast applied directly to a vector element misreads it)
    auto as_scalar = [](uint32_t bits) { return __builtin_bit_cast(Scalar, bits); };
    // (up to seven splits are read before the first add waits for one: the loop is otherwise
    // one memory round trip per split)
    u32x4 v = *reinterpret_cast<const u32x4*>(p);
    Scalar sum[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const uint32_t b = v[e];
      sum[e] = as_scalar(b);
    }
    for (int sp = 1; sp < splits; sp += 7) {
      u32x4 u[7];
#pragma unroll
      for (int i = 0; i < 7; ++i)
        if (sp + i < splits) u[i] = *reinterpret_cast<const u32x4*>(p + (sp + i) * split_stride);
#pragma unroll
      for (int i = 0; i < 7; ++i)
        if (sp + i < splits) {
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const uint32_t b = u[i][e];
            sum[e] += as_scalar(b);
          }
        }
    }
    epi(r, c, sum[0], sum[1], sum[2], sum[3]);
  }
}

// What a stage costs a workgroup of each operand layout (see tile_plan.h).
template <typename Math, int BMODE>
constexpr StageCost stage_cost() {
  if constexpr (BMODE == B_KN32) return STAGE_COST_KN32;
  if constexpr (BMODE == B_KN16) return STAGE_COST_KN16;
  if constexpr (BMODE == B_NK) return STAGE_COST_NK8;
  return STAGE_COST_KN8;
}

// An epilogue may declare `static constexpr bool REGISTER_HEAVY = true` to stay on the
// four-wave form of the 256-row tile (512 registers per wave instead of 256).
template <typename E, typename = void>
struct epi_register_heavy : std::false_type {};
template <typename E>
struct epi_register_heavy<E, typename std::enable_if<E::REGISTER_HEAVY>::type> : std::true_type {};

// The 256-row tile has two forms that fetch, multiply and store the same data in the same
// order (results identical bit for bit): four waves of 128 x 128, one per SIMD, and eight waves
// of 64 x 128, two per SIMD, where one wave's other instructions issue under the other's MFMAs,
// at 1.5 x the LDS fragment traffic.  Since the four-wave main loop carries no ring arithmetic
// (12-stage body, see `stage`) the second form has little left to hide, and the chip, power
// limited, answers its extra LDS traffic with a lower clock.  Alternating in one process on the
// bench's data: bf16 8192^3 -0.1..+0.3 % for four waves, int8 N x K 8192^3 +-0.3 %, bf16 4096^3
// (one round) +1.1 %, int8 N x K 4096^3 -> int32 +6.8 %; only N x K int8 weights with a 16-bit
// output keep the eight waves (2048 x 11008 x 4096 at M = 1024, one round: 44.0 against 44.8 us).
template <typename Math, int BMODE, typename Epi>
void launch_tile_256(cigemmContext* ctx, int64_t M, int64_t N, int64_t K_bytes, const void* A,
                     int64_t lda_bytes, const void* B, int64_t ldb_bytes, const Epi& epi,
                     int splits = 1) {
  if constexpr (BMODE == B_NK && Epi::OUT_BYTES == 2 && !epi_register_heavy<Epi>::value)
    launch_tile_mt<Math, BMODE, 2, Epi, 4>(ctx, M, N, K_bytes, A, lda_bytes, B, ldb_bytes, epi,
                                           splits);
  else
    launch_tile_mt<Math, BMODE, 4, Epi, 2>(ctx, M, N, K_bytes, A, lda_bytes, B, ldb_bytes, epi,
                                           splits);
}

// The 128-row tile has the same two forms (four waves of 64 x 128, eight of 32 x 128); with
// N x K int8 weights the second is 9 % faster (2048 x 11008 x 4096: 108 -> 98 us), with K x N
// operands 2 % slower (their transposing fragment reads are twice as many instructions).
template <typename Math, int BMODE, typename Epi>
void launch_tile_128(cigemmContext* ctx, int64_t M, int64_t N, int64_t K_bytes, const void* A,
                     int64_t lda_bytes, const void* B, int64_t ldb_bytes, const Epi& epi,
                     int splits = 1) {
  if constexpr (BMODE == B_NK && !epi_register_heavy<Epi>::value)
    launch_tile_mt<Math, BMODE, 1, Epi, 4>(ctx, M, N, K_bytes, A, lda_bytes, B, ldb_bytes, epi,
                                           splits);
  else
    launch_tile_mt<Math, BMODE, 2, Epi, 2>(ctx, M, N, K_bytes, A, lda_bytes, B, ldb_bytes, epi,
                                           splits);
}

template <typename Math, int BMODE, typename Epi>
void launch_tile_any_mt(cigemmContext* ctx, int mt, int64_t M, int64_t N, int64_t K_bytes,
                        const void* A, int64_t lda_bytes, const void* B, int64_t ldb_bytes,
                        const Epi& epi, int splits = 1) {
  if (mt == 4)
    launch_tile_256<Math, BMODE>(ctx, M, N, K_bytes, A, lda_bytes, B, ldb_bytes, epi, splits);
  else if (mt == 3)
    launch_tile_mt<Math, BMODE, 3>(ctx, M, N, K_bytes, A, lda_bytes, B, ldb_bytes, epi, splits);
  else if (mt == 2)
    launch_tile_128<Math, BMODE>(ctx, M, N, K_bytes, A, lda_bytes, B, ldb_bytes, epi, splits);
  else
    launch_tile_mt<Math, BMODE, 1>(ctx, M, N, K_bytes, A, lda_bytes, B, ldb_bytes, epi, splits);
}

// Runs one plan: tiles of 64*mt rows; with more than one K range the ranges go over
// blockIdx.y, partial sums to the workspace, then one reduction launch with the real epilogue.
// Returns true when it ran as such a pair of launches.
template <typename Math, int BMODE, typename Epi>
bool run_tile_plan(cigemmContext* ctx, int mt, int splits, int64_t M, int64_t N, int64_t K_bytes,
                   const void* A, int64_t lda_bytes, const void* B, int64_t ldb_bytes,
                   const Epi& epi) {
  if (splits <= 1) {
    launch_tile_any_mt<Math, BMODE>(ctx, mt, M, N, K_bytes, A, lda_bytes, B, ldb_bytes, epi);
    return false;
  }
  typedef typename Math::scalar_t scalar_t;
  const int cus = ctx->num_cus > 0 ? ctx->num_cus : 256;
  uint32_t* ws = static_cast<uint32_t*>(ctx->workspace);
  const EpiPartialX4 part{ws, N, M * N};
  launch_tile_any_mt<Math, BMODE>(ctx, mt, M, N, K_bytes, A, lda_bytes, B, ldb_bytes, part,
                                  splits);
  const int64_t quads = M * (N / 4);
  const unsigned grid = (unsigned)((quads + 255) / 256 < 4 * (int64_t)cus ? (quads + 255) / 256
                                                                          : 4 * (int64_t)cus);
  hipLaunchKernelGGL((splitk_reduce_kernel<scalar_t, Epi>), dim3(grid), dim3(256), 0, ctx->stream,
                     (int)M, (int)N, ctx->last_k_splits, ws, M * N, epi);
  return true;
}

// Chooses the tile height, and, when the last round of 256-row tiles would leave most of the
// chip idle, covers the columns of the full rounds with 256-row tiles and the remaining
// columns with a second launch of shorter tiles.  Epi::shift_cols(c) returns the epilogue of
// the sub-problem starting at column c.
// Returns true when the problem was run as a split-K pair of launches.
template <typename Math, int BMODE, typename Epi>
bool launch_tile(cigemmContext* ctx, int64_t M, int64_t N, int64_t K_bytes, const void* A,
                 int64_t lda_bytes, const void* B, int64_t ldb_bytes, const Epi& epi) {
  const int cus = ctx->num_cus > 0 ? ctx->num_cus : 256;
  if (ctx->force_tile_mt >= 1 && ctx->force_tile_mt <= 4) {
    // a plan imposed through the measurement library: as asked, but for K ranges the
    // workspace cannot hold
    int64_t range_stages = 0;
    int sp = k_ranges(K_bytes, ctx->force_tile_splits, &range_stages);
    if (sp > 1 && (!ctx->workspace ||
                   (size_t)sp * (size_t)M * (size_t)N * 4 > ctx->ws_partial_bytes))
      sp = 1;
    return run_tile_plan<Math, BMODE>(ctx, ctx->force_tile_mt, sp, M, N, K_bytes, A, lda_bytes, B,
                                      ldb_bytes, epi);
  }
  double single = 0;
  constexpr TileUnits units = BMODE == B_KN32 ? TILE_UNITS_F32 : TILE_UNITS;
  const int mt = best_mt(M, N, cus, &single, units);
  if (((M + BM - 1) / BM) * ((N + BN - 1) / BN) <= cus) {
    // At most one round of 256-row tiles: pick the tile height and the number of K ranges
    // together.
    const SmallPlan plan =
        plan_small(cus, ctx->workspace ? ctx->ws_partial_bytes : 0, M, N, K_bytes, Epi::OUT_BYTES,
                   stage_cost<Math, BMODE>(), K_bytes * N);
    return run_tile_plan<Math, BMODE>(ctx, plan.mt, plan.splits, M, N, K_bytes, A, lda_bytes, B,
                                      ldb_bytes, epi);
  }
  {
    // Several rounds.  When the tiles of the last round would leave much of the chip idle: the
    // columns that fill whole rounds of 256-row tiles first, the remaining columns as a second,
    // separately planned launch (which may split K).  Measured over 80 shapes with 5..24 row
    // tiles (M = 1280..6144, N = 4096..14336; bf16 and int8 N x K), the two launches issued from
    // the host: where this rule takes them +3..+22 % (1536 x 11008 x 4096 bf16 143 -> 117 us,
    // 3584 x 14336 x 4096 347 -> 314), at worst -3 %; the shapes it leaves alone would lose up
    // to 7 %.
    const int64_t tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
    if (tiles_m * tiles_n > cus && tiles_m <= cus) {
      const int64_t cols_per_round = cus / tiles_m;
      const int64_t full_cols = (tiles_n / cols_per_round) * cols_per_round;
      if (full_cols > 0 && full_cols < tiles_n) {
        const int64_t n1 = full_cols * BN, n2 = N - n1;
        double rest = 0;
        const int mt2 = best_mt(M, n2, cus, &rest, units);
        // (a tie stays with the single launch: int8 2048 x 11008 x 4096, 473 tiles of 192 rows in
        // two rounds against 256 tiles of 256 rows + 176 of 128 rows, alternating in one process:
        // 85.3 against 86.0 us)
        if (tile_plan_cost(M, n1, 4, cus, units) + rest < single * 0.97) {
          launch_tile_256<Math, BMODE>(ctx, M, n1, K_bytes, A, lda_bytes, B, ldb_bytes, epi);
          const int rows1 = ctx->last_tile_rows, waves1 = ctx->last_waves;
          const char* B2 = static_cast<const char*>(B) +
                           (BMODE == B_NK ? n1 * ldb_bytes : n1 * Math::ELEM_BYTES);
          bool split = false;
          if (tiles_m * ((n2 + BN - 1) / BN) <= cus) {
            const SmallPlan plan =
                plan_small(cus, ctx->workspace ? ctx->ws_partial_bytes : 0, M, n2, K_bytes,
                           Epi::OUT_BYTES, stage_cost<Math, BMODE>(), K_bytes * n2);
            split = run_tile_plan<Math, BMODE>(ctx, plan.mt, plan.splits, M, n2, K_bytes, A,
                                               lda_bytes, B2, ldb_bytes, epi.shift_cols(n1));
          } else {
            launch_tile_any_mt<Math, BMODE>(ctx, mt2, M, n2, K_bytes, A, lda_bytes, B2, ldb_bytes,
                                            epi.shift_cols(n1));
          }
          ctx->first_tile_rows = rows1;
          ctx->first_waves = waves1;
          return split;
        }
      }
    }
  }
  launch_tile_any_mt<Math, BMODE>(ctx, mt, M, N, K_bytes, A, lda_bytes, B, ldb_bytes, epi);
  return false;
}

// Shape / alignment gate shared by the families (sizes in elements, elem = bytes each;
// b_kn = B is K x N).  M is free; K must fill whole 16-byte pieces (a last stage of fewer
// than four is completed with zeros); N a multiple of 4 (a last 16-byte piece of a K x N row
// that is only partly inside the matrix is still read whole: its row is 16-byte aligned, so the
// piece cannot leave the page that holds its first byte).  Per-lane DMA offsets are 32-bit: 256
// rows of either operand must span less than 2 GiB.
inline bool tile_shape_ok(int64_t M, int64_t N, int64_t K, int elem, const void* A, int64_t lda,
                          const void* B, int64_t ldb, bool b_kn) {
  if (M <= 0 || N <= 0 || K <= 0) return false;
  if ((K * elem) % 16 || N % 4) return false;
  if (M > 2147483647LL || N > 2147483647LL) return false;
  if ((lda * elem) % 16 || (ldb * elem) % 16) return false;
  if (((uintptr_t)A & 15) || ((uintptr_t)B & 15)) return false;
  if (((M + 63) / 64) * ((N + BN - 1) / BN) > 2147483647LL) return false;
  if (lda * elem * 256 >= (1LL << 31) || ldb * elem * 256 >= (1LL << 31)) return false;
  return true;
}

// The int8 tile kernels' gate: the shape gate above plus what their epilogues store in 16-byte
// pieces (output rows, the accumulator dump) or load as such (per-column scales).
inline bool i8_tile_ok(int64_t M, int64_t N, int64_t K, const int8_t* A, int64_t lda,
                       const int8_t* B, int64_t ldb, bool b_nk, const int32_t* C, int64_t ldc,
                       const DequantArgs* dq) {
  if (!tile_shape_ok(M, N, K, 1, A, lda, B, ldb, !b_nk)) return false;
  if (!dq) {
    if (ldc % 4 || ((uintptr_t)C & 15)) return false;
  } else {
    if (dq->ldo % (dq->out_bf16 ? 8 : 4) || ((uintptr_t)dq->out & 15)) return false;
    if (dq->sb_vec && ((uintptr_t)dq->sb & 15)) return false;
    if (dq->acc_out && (dq->ldacc % 4 || ((uintptr_t)dq->acc_out & 15))) return false;
  }
  return true;
}

}  // namespace tile
}  // namespace cig
