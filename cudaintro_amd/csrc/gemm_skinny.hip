// Skinny (decode-shape) GEMMs: y[M x N] = x[M x K] . W with M <= 32.  The weights are read
// once and nothing is reused, so these kernels are bound by HBM bandwidth; they exist to keep
// a deep, wide stream of weight bytes in flight, not to save arithmetic.
//
// Workgroup = 256 lanes = 4 waves; it owns BN output columns and one K range (split-K), and
// walks its K range in stages held in a ring in LDS (7 or 8 stages, 140-144 KiB): one stage =
// one weight tile (16 KiB) + the matching slice of x, all moved by LDS-DMA, NSTAGES-1 stages
// in flight.  The arithmetic is the 32x32 MFMA with x padded to 32 rows (rows >= M re-read
// row M-1 and are never stored): at M <= 32 the matrix core is idle most of the time anyway.
//
//   16-bit, W is K x N (n contiguous):  BN = 256, stage = 32 k: W tile [32 k][256 n] read back
//       with the transposing LDS read (same layout as the big tile kernel), x tile [32 m][64 B].
//   int8, W is N x K (k contiguous):    BN = 128, stage = 128 k: W tile [128 n][128 B],
//       x tile [32 m][128 B], both read with 16-byte LDS reads.
//
// Split-K: each workgroup writes its 32 x BN partial (fp32 / int32) to the handle's
// workspace, then bumps a per-column-slab counter; the workgroup that finds it is the last
// one sums the partials in split order (so the result does not depend on arrival order),
// applies the epilogue and resets the counter.
//
// int8 weights with at least one 32-column slab per compute unit take a second kernel that
// needs none of that: K is split over the four waves of the workgroup (further down).
// K x N weights (16-bit, int8) with N and K multiples of 64 (int8: 128) take a third one: slabs
// of one or two whole 128-byte lines per weight row, K over the waves, short rings so that two
// workgroups fit a compute unit (further down; it serves nearly every 16-bit decode shape).
#include <atomic>
#include <cstdarg>
#include <mutex>

#include "epilogues.h"
#include "mfma_tile.h"
#include "skinny_plan.h"

namespace cig {
namespace {

using tile::lds_void;

constexpr int XROWS = 32;  // x padded to one MFMA tile of rows

__device__ __forceinline__ void dma16(const char* src, uint32_t lds_dst) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off"
               :
               : "s"(lds_dst), "v"(src)
               : "m0");
}
__device__ __forceinline__ void dma4(const char* src, uint32_t lds_dst) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, off"
               :
               : "s"(lds_dst), "v"(src)
               : "m0");
}

// s_waitcnt vmcnt(n), everything else unconstrained: vmcnt is split over bits 3:0 and 15:14.
template <int N>
__device__ __forceinline__ void wait_vmcnt_n() {
  static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
  __builtin_amdgcn_s_waitcnt(0x0f70 | (N & 15) | ((N >> 4) << 14));
}
// Waits until at most `rem` stages of PER_STAGE DMA instructions each are still in flight
// (rem <= MAX_REM; the count of s_waitcnt is an immediate, hence the switch).
template <int PER_STAGE, int MAX_REM>
__device__ __forceinline__ void wait_stages_in_flight(int rem) {
  static_assert(MAX_REM <= 15 && PER_STAGE * MAX_REM < 64, "vmcnt is a 6-bit counter");
#define CIG_WAIT_CASE(R) \
  case R: wait_vmcnt_n<PER_STAGE * (MAX_REM >= R ? R : 0)>(); break;
  switch (rem) {
    CIG_WAIT_CASE(0) CIG_WAIT_CASE(1) CIG_WAIT_CASE(2) CIG_WAIT_CASE(3) CIG_WAIT_CASE(4)
    CIG_WAIT_CASE(5) CIG_WAIT_CASE(6) CIG_WAIT_CASE(7) CIG_WAIT_CASE(8) CIG_WAIT_CASE(9)
    CIG_WAIT_CASE(10) CIG_WAIT_CASE(11) CIG_WAIT_CASE(12) CIG_WAIT_CASE(13) CIG_WAIT_CASE(14)
    default: wait_vmcnt_n<PER_STAGE * MAX_REM>(); break;
  }
#undef CIG_WAIT_CASE
}

// ---- 16-bit weights, K x N ------------------------------------------------------------------
template <typename MathT>
struct GeoKN16 {
  typedef MathT Math;
  typedef tile::BTile<tile::B_KN16> WT;
  static constexpr int BN = 256;
  static constexpr int K_ELEMS = 32;                 // k per stage
  static constexpr int W_BYTES = 32 * 512;           // [32 k][256 n] halves
  static constexpr int X_BYTES = XROWS * 64;         // [32 m][64 B]
  static constexpr int STAGE_BYTES = W_BYTES + X_BYTES;
  static constexpr int NSTAGES = 8;                  // 144 KiB
  static constexpr int DMA_PER_STAGE = 6;            // per wave: 4 W (1 KiB) + 2 x (256 B)
  static constexpr int NT = 2;                       // 32-column tiles per wave

  // W points at (k = first k of the stage, n = n0); x at (row 0, same k), both in bytes.
  static __device__ __forceinline__ void dma(const char* W, int64_t ldw, const char* x, int64_t ldx,
                                             int M, uint32_t slot_lds, int w, int l) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
      dma16(W + WT::dma_src(w, i, l, ldw, 31), slot_lds + WT::dma_lds(w, i));
    // x: only the groups of four rows that hold a row below M (the other rows of the padded
    // tile keep whatever the LDS holds: their products are never stored)
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      if (8 * w + 4 * i < M) {
        const int r = 8 * w + 4 * i + (l >> 4);
        const int rr = r < M ? r : M - 1;
        const int chunk = ((l & 15) >> 2) ^ tile::rowmajor_swz(r);
        dma4(x + (int64_t)rr * ldx + (chunk << 4) + ((l & 3) << 2),
             slot_lds + W_BYTES + (8 * w + 4 * i) * 64);
      }
    }
  }
  // DMA instructions wave w issues per stage
  static __device__ __forceinline__ int dma_count(int M, int w) {
    return 4 + (8 * w < M ? 1 : 0) + (8 * w + 4 < M ? 1 : 0);
  }
  static __device__ __forceinline__ void compute(const char* slot, int w, int l,
                                                 typename Math::acc_t (&acc)[NT]) {
    const char* sx = slot + W_BYTES;
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
      const u32x4 xf =
          *reinterpret_cast<const u32x4*>(sx + tile::rowmajor_off(l & 31, 2 * kk + (l >> 5)));
#pragma unroll
      for (int j = 0; j < NT; ++j) {
        const u32x2 lo = WT::frag_half(slot, 0, 2 * w + j, kk, 0, l);
        const u32x2 hi = WT::frag_half(slot, 0, 2 * w + j, kk, 1, l);
        acc[j] = Math::mfma(__builtin_shufflevector(lo, hi, 0, 1, 2, 3), xf, acc[j]);
      }
    }
  }
  // first column (relative to n0) of accumulator quad q of tile j
  static __device__ __forceinline__ int col(int w, int j, int q, int l) {
    return 64 * w + 32 * j + 8 * q + 4 * (l >> 5);
  }
  static __device__ __forceinline__ int64_t w_stage_step(int64_t ldw) { return 32 * ldw; }
  static constexpr int X_STAGE_STEP = 64;
};

// ---- int8 weights, N x K ----------------------------------------------------------------------
struct GeoNK8 {
  typedef tile::MathI8 Math;
  static constexpr int BN = 128;
  static constexpr int K_ELEMS = 128;
  static constexpr int W_BYTES = 128 * 128;          // [128 n][128 B]
  static constexpr int X_BYTES = XROWS * 128;        // [32 m][128 B]
  static constexpr int STAGE_BYTES = W_BYTES + X_BYTES;
  static constexpr int NSTAGES = 7;                  // 140 KiB
  static constexpr int DMA_PER_STAGE = 5;            // per wave: 4 W + 1 x, 1 KiB each
  static constexpr int NT = 1;

  // 128-byte rows, 8 chunks: chunk c of row r at r*128 + ((c ^ swz(r)) << 4)
  static __device__ __forceinline__ int swz(int r) { return ((r >> 1) & 7) ^ ((r & 1) << 2); }
  static __device__ __forceinline__ int off(int r, int c) { return r * 128 + ((c ^ swz(r)) << 4); }

  static __device__ __forceinline__ void dma(const char* W, int64_t ldw, const char* x, int64_t ldx,
                                             int M, uint32_t slot_lds, int w, int l) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int r = 32 * w + 8 * i + (l >> 3);
      dma16(W + (int64_t)r * ldw + (((l & 7) ^ swz(r)) << 4), slot_lds + (32 * w + 8 * i) * 128);
    }
    // x: only the groups of eight rows that hold a row below M (see above)
    if (8 * w < M) {
      const int r = 8 * w + (l >> 3);
      const int rr = r < M ? r : M - 1;
      dma16(x + (int64_t)rr * ldx + (((l & 7) ^ swz(r)) << 4), slot_lds + W_BYTES + (8 * w) * 128);
    }
  }
  static __device__ __forceinline__ int dma_count(int M, int w) { return 4 + (8 * w < M ? 1 : 0); }
  static __device__ __forceinline__ void compute(const char* slot, int w, int l,
                                                 Math::acc_t (&acc)[NT]) {
    const char* sx = slot + W_BYTES;
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
      const u32x4 xf = *reinterpret_cast<const u32x4*>(sx + off(l & 31, 2 * kk + (l >> 5)));
      const u32x4 wf =
          *reinterpret_cast<const u32x4*>(slot + off(32 * w + (l & 31), 2 * kk + (l >> 5)));
      acc[0] = Math::mfma(wf, xf, acc[0]);
    }
  }
  static __device__ __forceinline__ int col(int w, int j, int q, int l) {
    return 32 * w + 8 * q + 4 * (l >> 5);
  }
  static __device__ __forceinline__ int64_t w_stage_step(int64_t) { return 128; }
  static constexpr int X_STAGE_STEP = 128;
};

template <typename Geo>
__device__ __forceinline__ const char* w_origin(const char* W, int64_t ldw, int64_t n0,
                                                int64_t k0_elems);
template <>
__device__ __forceinline__ const char* w_origin<GeoNK8>(const char* W, int64_t ldw, int64_t n0,
                                                        int64_t k0) {
  return W + n0 * ldw + k0;
}
template <typename Geo>
__device__ __forceinline__ const char* w_origin(const char* W, int64_t ldw, int64_t n0,
                                                int64_t k0) {
  return W + k0 * ldw + n0 * 2;  // K x N halves
}

// Partials cross workgroups on different XCDs, each with its own L2, so they are written
// and read with agent-scope accesses (which go through to the coherence point) rather than
// ordinary cached ones plus an agent-scope fence: that fence writes back and invalidates the
// whole L2 and costs tens of microseconds per call.  A quad of partial sums travels as two
// 64-bit words; the layout is private to this kernel and lane-contiguous
// ([split][slab][quad][half][lane]) so every access instruction moves 512 contiguous bytes.
template <typename T>
__device__ __forceinline__ void store_partial(uint64_t* dst, T v0, T v1, T v2, T v3) {
  const uint64_t lo = (uint64_t)__builtin_bit_cast(uint32_t, v0) |
                      ((uint64_t)__builtin_bit_cast(uint32_t, v1) << 32);
  const uint64_t hi = (uint64_t)__builtin_bit_cast(uint32_t, v2) |
                      ((uint64_t)__builtin_bit_cast(uint32_t, v3) << 32);
  __hip_atomic_store(dst, lo, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __hip_atomic_store(dst + 256, hi, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// The reduction of the last workgroup of a slab: NQ quads of this thread, summed over the S
// partial tiles in split order, each sum starting from zero (the result does not depend on which
// workgroup arrived last).  `first` = word of (split 0, this slab, quad 0, half 0, this lane),
// `split_stride` = words between the tiles of consecutive splits.  The loads of up to 32 quads
// are issued back to back before the first sum waits: a load from the coherence point takes
// most of a microsecond, and one round trip per quad and split was a third of the time of a
// 16 MB weight matrix.
template <typename T, int NQ, int S>
__device__ __forceinline__ void sum_partials(const uint64_t* first, int64_t split_stride,
                                             T (&sum)[NQ][4]) {
  constexpr int CH = S * NQ <= 32 ? S : (32 / NQ > 0 ? 32 / NQ : 1);  // splits per batch
#pragma unroll
  for (int q = 0; q < NQ; ++q)
#pragma unroll
    for (int e = 0; e < 4; ++e) sum[q][e] = 0;
#pragma unroll
  for (int s0 = 0; s0 < S; s0 += CH) {
    uint64_t lo[CH][NQ], hi[CH][NQ];
#pragma unroll
    for (int c = 0; c < CH; ++c)
#pragma unroll
      for (int q = 0; q < NQ; ++q) {
        const uint64_t* src = first + (s0 + c) * split_stride + q * 512;
        lo[c][q] = __hip_atomic_load(src, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        hi[c][q] = __hip_atomic_load(src + 256, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
#pragma unroll
    for (int c = 0; c < CH; ++c)
#pragma unroll
      for (int q = 0; q < NQ; ++q) {
        sum[q][0] += __builtin_bit_cast(T, (uint32_t)lo[c][q]);
        sum[q][1] += __builtin_bit_cast(T, (uint32_t)(lo[c][q] >> 32));
        sum[q][2] += __builtin_bit_cast(T, (uint32_t)hi[c][q]);
        sum[q][3] += __builtin_bit_cast(T, (uint32_t)(hi[c][q] >> 32));
      }
  }
}

// The same for a number of K ranges known only at run time (up to 16): batches of up to 32 quads
// whose loads are issued back to back under uniform conditions.
template <typename T, int NQ>
__device__ __forceinline__ void sum_partials_n(const uint64_t* first, int64_t split_stride,
                                               int splits, T (&sum)[NQ][4]) {
  constexpr int CH = 32 / NQ > 0 ? 32 / NQ : 1;  // splits per batch
#pragma unroll
  for (int q = 0; q < NQ; ++q)
#pragma unroll
    for (int e = 0; e < 4; ++e) sum[q][e] = 0;
#pragma unroll
  for (int s0 = 0; s0 < 16; s0 += CH) {
    if (s0 >= splits) break;
    uint64_t lo[CH][NQ], hi[CH][NQ];
#pragma unroll
    for (int c = 0; c < CH; ++c)
      if (s0 + c < splits) {
#pragma unroll
        for (int q = 0; q < NQ; ++q) {
          const uint64_t* src = first + (s0 + c) * split_stride + q * 512;
          lo[c][q] = __hip_atomic_load(src, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          hi[c][q] = __hip_atomic_load(src + 256, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
      }
#pragma unroll
    for (int c = 0; c < CH; ++c)
      if (s0 + c < splits) {
#pragma unroll
        for (int q = 0; q < NQ; ++q) {
          sum[q][0] += __builtin_bit_cast(T, (uint32_t)lo[c][q]);
          sum[q][1] += __builtin_bit_cast(T, (uint32_t)(lo[c][q] >> 32));
          sum[q][2] += __builtin_bit_cast(T, (uint32_t)hi[c][q]);
          sum[q][3] += __builtin_bit_cast(T, (uint32_t)(hi[c][q] >> 32));
        }
      }
  }
}

// Workspace: the partials (see store_partial) followed by one arrival counter per slab.
template <typename Geo, typename Epi, int SPLITS>
__global__ __launch_bounds__(256, 1) void skinny_kernel(int M, int N, int stages_per_split,
                                                        const char* __restrict__ X,
                                                        int64_t ldx, const char* __restrict__ W,
                                                        int64_t ldw, Epi epi,
                                                        uint64_t* __restrict__ partials,
                                                        uint32_t* __restrict__ counters) {
  typedef typename Geo::Math Math;
  typedef typename Math::acc_t acc_t;
  typedef typename Math::scalar_t scalar_t;
  constexpr int NS = Geo::NSTAGES, DIST = NS - 1, DPS = Geo::DMA_PER_STAGE;
  extern __shared__ __attribute__((aligned(1024))) char lds[];
  __shared__ int is_last;
  const int t = threadIdx.x, l = t & 63;
  const int w = __builtin_amdgcn_readfirstlane(t >> 6);
  constexpr int splits = SPLITS;
  const int slab = blockIdx.x / splits, split = blockIdx.x % splits;
  const int64_t n0 = (int64_t)slab * Geo::BN;
  const int64_t k0 = (int64_t)split * stages_per_split * Geo::K_ELEMS;
  const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)lds;

  const char* w_src = w_origin<Geo>(W, ldw, n0, k0);
  const char* x_src = X + k0 * Math::ELEM_BYTES;
  const int64_t w_step = Geo::w_stage_step(ldw);
  const int KTS = stages_per_split;

  auto issue = [&](int st, int slot) {
    Geo::dma(w_src + st * w_step, ldw, x_src + (int64_t)st * Geo::X_STAGE_STEP, ldx, M,
             lds_base + slot * Geo::STAGE_BYTES, w, l);
  };

  acc_t acc[Geo::NT];
#pragma unroll
  for (int j = 0; j < Geo::NT; ++j)
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[j][e] = 0;

#pragma unroll
  for (int st = 0; st < DIST; ++st)
    if (st < KTS) issue(st, st);

  // this wave's DMA instructions per stage: the W pieces plus the x pieces below row M
  const int dps = Geo::dma_count(M, w);
  int slot = 0, dma_slot = DIST;
  for (int s = 0; s < KTS; ++s) {
    // Stage s landed for this wave; the stages after it that have been issued (at most
    // DIST - 1, fewer at the end of the K range: nothing is fetched past it) may be in flight.
    // After the barrier stage s is visible to all waves and every wave has finished reading
    // stage s - 1.
    const int rem = KTS - 1 - s < DIST - 1 ? KTS - 1 - s : DIST - 1;
    if (dps == DPS)
      wait_stages_in_flight<DPS, DIST - 1>(rem);
    else if (dps == DPS - 1)
      wait_stages_in_flight<DPS - 1, DIST - 1>(rem);
    else
      wait_stages_in_flight<DPS - 2, DIST - 1>(rem);
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
    if (s + DIST < KTS) issue(s + DIST, dma_slot);
    Geo::compute(lds + slot * Geo::STAGE_BYTES, w, l, acc);
    slot = slot + 1 == NS ? 0 : slot + 1;
    dma_slot = dma_slot + 1 == NS ? 0 : dma_slot + 1;
  }

  const int m = l & 31;
  if (splits == 1) {
    if (m < M) {
#pragma unroll
      for (int j = 0; j < Geo::NT; ++j)
#pragma unroll
        for (int q = 0; q < 4; ++q)
          epi(m, n0 + Geo::col(w, j, q, l), acc[j][4 * q], acc[j][4 * q + 1], acc[j][4 * q + 2],
              acc[j][4 * q + 3]);
    }
    return;
  }

  // ---- split-K: publish the partial, last workgroup of the slab reduces in split order -------
  constexpr int QUADS = Geo::NT * 4;
  const int slabs = gridDim.x / splits;
  // 64-bit word index of (split sp, this slab, quad 0, half 0, this lane)
  auto part = [&](int sp) {
    return partials + ((int64_t)(sp * slabs + slab) * QUADS * 2) * 256 + t;
  };
  if (m < M) {
    uint64_t* dst = part(split);
#pragma unroll
    for (int j = 0; j < Geo::NT; ++j)
#pragma unroll
      for (int q = 0; q < 4; ++q)
        store_partial(dst + (j * 4 + q) * 512, acc[j][4 * q], acc[j][4 * q + 1],
                      acc[j][4 * q + 2], acc[j][4 * q + 3]);
  }
  // every lane's partial stores have been acknowledged before the arrival is counted
  __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0)
  __syncthreads();
  if (t == 0) {
    const uint32_t old = __hip_atomic_fetch_add(counters + slab, 1u, __ATOMIC_RELAXED,
                                                __HIP_MEMORY_SCOPE_AGENT);
    is_last = old == (uint32_t)(splits - 1);
  }
  __syncthreads();
  if (!is_last) return;
  if (m < M) {
    scalar_t sum[QUADS][4];
    sum_partials<scalar_t, QUADS, splits>(part(0), (int64_t)slabs * QUADS * 512, sum);
#pragma unroll
    for (int j = 0; j < Geo::NT; ++j)
#pragma unroll
      for (int q = 0; q < 4; ++q)
        epi(m, n0 + Geo::col(w, j, q, l), sum[4 * j + q][0], sum[4 * j + q][1], sum[4 * j + q][2],
            sum[4 * j + q][3]);
  }
  if (t == 0) __hip_atomic_store(counters + slab, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Number of K splits: skinny_plan.h has the rule.
template <typename Geo>
int choose_splits(const cigemmContext* ctx, int64_t N, int64_t kts) {
  return skinny_plan::barrier_kernel_splits(N / Geo::BN, N, kts, XROWS, ctx->num_cus,
                                            ctx->ws_counter_bytes, ctx->ws_partial_bytes);
}

template <typename Geo, typename Epi, int SPLITS>
void launch_skinny_n(cigemmContext* ctx, int64_t M, int64_t N, int64_t kts, const void* X,
                     int64_t ldx_bytes, const void* W, int64_t ldw_bytes, const Epi& epi) {
  constexpr int LDS_BYTES = Geo::NSTAGES * Geo::STAGE_BYTES;
  auto kern = skinny_kernel<Geo, Epi, SPLITS>;
  static std::atomic<uint64_t> lds_set{0};
  if (!ensure_dynamic_lds(ctx, (const void*)kern, LDS_BYTES, lds_set)) return;
  const unsigned grid = (unsigned)((N / Geo::BN) * SPLITS);
  hipLaunchKernelGGL(kern, dim3(grid), dim3(256), LDS_BYTES, ctx->stream, (int)M, (int)N,
                     (int)(kts / SPLITS), static_cast<const char*>(X), ldx_bytes,
                     static_cast<const char*>(W), ldw_bytes, epi,
                     static_cast<uint64_t*>(ctx->workspace),
                     reinterpret_cast<uint32_t*>(static_cast<char*>(ctx->workspace) +
                                                 ctx->ws_partial_bytes));
}

template <typename Geo, typename Epi>
void launch_skinny(cigemmContext* ctx, int64_t M, int64_t N, int64_t K, const void* X,
                   int64_t ldx_bytes, const void* W, int64_t ldw_bytes, const Epi& epi) {
  const int64_t kts = K / Geo::K_ELEMS;
  switch (choose_splits<Geo>(ctx, N, kts)) {
    case 16: launch_skinny_n<Geo, Epi, 16>(ctx, M, N, kts, X, ldx_bytes, W, ldw_bytes, epi); break;
    case 8: launch_skinny_n<Geo, Epi, 8>(ctx, M, N, kts, X, ldx_bytes, W, ldw_bytes, epi); break;
    case 4: launch_skinny_n<Geo, Epi, 4>(ctx, M, N, kts, X, ldx_bytes, W, ldw_bytes, epi); break;
    case 2: launch_skinny_n<Geo, Epi, 2>(ctx, M, N, kts, X, ldx_bytes, W, ldw_bytes, epi); break;
    default: launch_skinny_n<Geo, Epi, 1>(ctx, M, N, kts, X, ldx_bytes, W, ldw_bytes, epi); break;
  }
}

// ---- int8, N x K weights, many columns: no split-K ------------------------------------------
// With at least one 32-column slab per compute unit the K split moves inside the workgroup:
// a stage is 512 k of the slab's 32 weight rows (16 KiB, 512 contiguous bytes per row) plus
// the same 512 k of XR rows of x (XR = 8, 16 or 32, the smallest that holds M); wave w moves
// and multiplies k-chunk w (128 k) of every stage, and the four partial 32 x 32 tiles are
// summed through LDS in wave order at the end.  No partials in memory, no arrival counter, no
// second pass: the three dependent trips through the fabric that the split-K fix-up costs
// (about 5 us per call) are gone.
template <int XR_, bool DEEP_ = false>
struct NK8KW {
  static constexpr int BN = 32;
  static constexpr int K_ELEMS = 512;
  static constexpr int XR = XR_;                     // rows of x held per stage
  static constexpr int W_BYTES = 32 * 512;           // four [32 n][128 B] sub-tiles, one per wave
  static constexpr int X_BYTES = XR * 512;           // four [XR m][128 B] sub-tiles
  static constexpr int STAGE_BYTES = W_BYTES + X_BYTES;
  // Two workgroups share the LDS of a compute unit (60 / 72 / 64 KiB each): with more slabs
  // than units nobody waits for a second round, and with fewer the shallower ring is no slower
  // (M = 8: N = K = 8192 13.9 -> 13.1 us, 11008 x 4096 15.1 -> 12.7, 28672 x 8192 47.8 ->
  // 43.1).  With 32 rows of x only two stages fit beside a second workgroup, and that ring is
  // slower when a workgroup has its unit to itself (N = K = 8192: 14.8 -> 16.4 us), faster with
  // more slabs than units (16384 x 4096: 19.9 -> 15.2): DEEP_ is the ring of 5 stages (160 KiB,
  // one workgroup per unit) for the first case.
  static constexpr int NSTAGES = DEEP_ ? 5 : XR == 32 ? 2 : 3;
  static constexpr int DPS = 4 + XR / 8;             // per wave and stage, 1 KiB each
};

template <typename Epi, int XR, bool DEEP, bool ROW_TILES>
__global__ __launch_bounds__(256, 2) void skinny_nk8_kwaves_kernel(int M, int N, int K,
                                                                   const char* __restrict__ X,
                                                                   int64_t ldx,
                                                                   const char* __restrict__ W,
                                                                   int64_t ldw, Epi epi,
                                                                   int row_tiles) {
  typedef tile::MathI8 Math;
  typedef NK8KW<XR, DEEP> G;
  constexpr int NS = G::NSTAGES, DIST = NS - 1;
  extern __shared__ __attribute__((aligned(1024))) char lds[];
  const int t = threadIdx.x, l = t & 63;
  const int w = __builtin_amdgcn_readfirstlane(t >> 6);
  // With several row tiles the grid is that many times the slabs: rows 0 .. XR - 1, XR .. 2 XR - 1,
  // ... of x go to different workgroups, which the block order puts on the same XCD (blocks b,
  // b + 8, ...) and close in time, so that the later ones find the slab's weight rows in that
  // XCD's L2.
  int slab = blockIdx.x, m_base = 0;
  if constexpr (ROW_TILES) {
    if (gridDim.x % (8 * row_tiles) == 0) {
      m_base = ((blockIdx.x >> 3) % row_tiles) * XR;
      slab = blockIdx.x / (8 * row_tiles) * 8 + (blockIdx.x & 7);
    } else {
      m_base = (blockIdx.x % row_tiles) * XR;
      slab = blockIdx.x / row_tiles;
    }
    if (m_base >= M) return;  // (a tile past the last row: nothing to do)
    X += (int64_t)m_base * ldx;
    M = M - m_base < XR ? M - m_base : XR;
  }
  const int64_t n0 = (int64_t)slab * G::BN;
  const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)lds;
  // K is a multiple of 128: the last stage may hold fewer than four k-chunks
  const int KTS = (K + G::K_ELEMS - 1) / G::K_ELEMS;

  // this lane's DMA sources at k = 0: row 8 i + l / 8 of the slab (i = 0..3) and of x
  // (i < XR / 8; rows >= M re-read row M - 1), 16-byte chunk (l % 8) ^ swz(row) of a k-chunk
  const char* wsrc[4];
  const char* xsrc[XR / 8];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = 8 * i + (l >> 3);
    wsrc[i] = W + (n0 + r) * ldw + (((l & 7) ^ GeoNK8::swz(r)) << 4);
    if (i < XR / 8)
      xsrc[i] = X + (int64_t)(r < M ? r : M - 1) * ldx + (((l & 7) ^ GeoNK8::swz(r)) << 4);
  }
  // Workgroups start at different stages of K and wrap around (integer sums do not depend on
  // the order): at any moment they read different 512-byte columns of their rows, which spreads
  // the requests over the memory channels (19.4 -> 14.1 us per call at N = K = 8192).
  const int rot = (int)(((unsigned)slab * 7u) % (unsigned)KTS);
  // first k of wave w's chunk of the s-th stage this workgroup visits, or -1 when that chunk
  // lies past K (last stage of a K that is not a multiple of 512)
  auto chunk_k = [&](int s) {
    int st = s + rot;
    st = st < KTS ? st : st - KTS;
    const int k = st * G::K_ELEMS + 128 * w;
    return k < K ? k : -1;
  };
  // Past the last stage the last one is fetched again into a slot nobody reads any more: the
  // number of instructions in flight, and so the wait count, stays the same to the end
  // (measured against issuing nothing past the end and waiting for exactly what is in flight:
  // 14.1 against 14.7 us at M = 1, N = K = 8192).
  auto issue = [&](int s, int slot) {
    s = s < KTS ? s : KTS - 1;
    int k = chunk_k(s);
    k = k >= 0 ? k : K - 128;   // a chunk past K: fetch the last valid one, never multiplied
    const uint32_t dst = lds_base + slot * G::STAGE_BYTES;
#pragma unroll
    for (int i = 0; i < 4; ++i) dma16(wsrc[i] + k, dst + w * 4096 + (8 * i) * 128);
#pragma unroll
    for (int i = 0; i < XR / 8; ++i)
      dma16(xsrc[i] + k, dst + G::W_BYTES + w * (XR * 128) + (8 * i) * 128);
  };

  Math::acc_t acc;
#pragma unroll
  for (int e = 0; e < 16; ++e) acc[e] = 0;
#pragma unroll
  for (int st = 0; st < DIST; ++st) issue(st, st);

  int slot = 0, dma_slot = DIST;
  for (int s = 0; s < KTS; ++s) {
    // Stage s landed for this wave.  No workgroup barrier: a wave reads only the k-chunk it
    // moved itself, and the slot it refills now is the one of stage s - 1, whose fragments
    // its own MFMAs have already consumed.
    wait_vmcnt_n<G::DPS*(DIST - 1)>();
    __builtin_amdgcn_sched_barrier(0);
    issue(s + DIST, dma_slot);
    const char* sw = lds + slot * G::STAGE_BYTES + w * 4096;
    const char* sx = lds + slot * G::STAGE_BYTES + G::W_BYTES + w * (XR * 128);
    if (chunk_k(s) >= 0) {
#pragma unroll
      for (int kk = 0; kk < 4; ++kk) {
        // rows XR .. 31 of the padded x tile alias rows 0 .. XR - 1: never stored
        const u32x4 xf =
            *reinterpret_cast<const u32x4*>(sx + GeoNK8::off(l & (XR - 1), 2 * kk + (l >> 5)));
        const u32x4 wf =
            *reinterpret_cast<const u32x4*>(sw + GeoNK8::off(l & 31, 2 * kk + (l >> 5)));
        acc = Math::mfma(wf, xf, acc);
      }
    }
    slot = slot + 1 == NS ? 0 : slot + 1;
    dma_slot = dma_slot + 1 == NS ? 0 : dma_slot + 1;
  }
  wait_vmcnt_n<0>();
  __syncthreads();  // no DMA in flight, every wave done reading: the ring can be reused

  // acc[4 q + e] = partial of y[l % 32][n0 + 8 q + 4 (l / 32) + e] over this wave's k-chunks
  int32_t* red = reinterpret_cast<int32_t*>(lds);  // [4 waves][32 m][36]
  constexpr int RLD = 36;
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const i32x4 v = {acc[4 * q], acc[4 * q + 1], acc[4 * q + 2], acc[4 * q + 3]};
    *reinterpret_cast<i32x4*>(red + (w * 32 + (l & 31)) * RLD + 8 * q + 4 * (l >> 5)) = v;
  }
  __syncthreads();
  const int m = t >> 3, c = (t & 7) * 4;
  if (m >= M) return;
  i32x4 sum = *reinterpret_cast<const i32x4*>(red + m * RLD + c);
#pragma unroll
  for (int ww = 1; ww < 4; ++ww) {
    const i32x4 p = *reinterpret_cast<const i32x4*>(red + (ww * 32 + m) * RLD + c);
    sum += p;
  }
  epi(m + m_base, n0 + c, sum[0], sum[1], sum[2], sum[3]);
}

template <typename Epi, int XR, bool DEEP>
void launch_skinny_kwaves_ring(cigemmContext* ctx, int64_t M, int64_t N, int64_t K, const void* X,
                               int64_t ldx_bytes, const void* W, int64_t ldw_bytes,
                               const Epi& epi) {
  typedef NK8KW<XR, DEEP> G;
  constexpr int LDS_BYTES = G::NSTAGES * G::STAGE_BYTES;
  static_assert(LDS_BYTES * (DEEP ? 1 : 2) <= 160 * 1024, "rings must fit the LDS");
  auto kern = skinny_nk8_kwaves_kernel<Epi, XR, DEEP, false>;
  static std::atomic<uint64_t> lds_set{0};
  if (!ensure_dynamic_lds(ctx, (const void*)kern, LDS_BYTES, lds_set)) return;
  hipLaunchKernelGGL(kern, dim3((unsigned)(N / G::BN)), dim3(256), LDS_BYTES, ctx->stream, (int)M,
                     (int)N, (int)K, static_cast<const char*>(X), ldx_bytes,
                     static_cast<const char*>(W), ldw_bytes, epi, 1);
}

// the same with the rows of x cut into `row_tiles` tiles of XR rows (nk8_row_tiles)
template <typename Epi, int XR>
void launch_skinny_kwaves_row_tiles(cigemmContext* ctx, int64_t M, int64_t N, int64_t K,
                                    const void* X, int64_t ldx_bytes, const void* W,
                                    int64_t ldw_bytes, const Epi& epi, int row_tiles) {
  typedef NK8KW<XR, false> G;
  constexpr int LDS_BYTES = G::NSTAGES * G::STAGE_BYTES;
  auto kern = skinny_nk8_kwaves_kernel<Epi, XR, false, true>;
  static std::atomic<uint64_t> lds_set{0};
  if (!ensure_dynamic_lds(ctx, (const void*)kern, LDS_BYTES, lds_set)) return;
  hipLaunchKernelGGL(kern, dim3((unsigned)(N / G::BN * row_tiles)), dim3(256), LDS_BYTES,
                     ctx->stream, (int)M, (int)N, (int)K, static_cast<const char*>(X), ldx_bytes,
                     static_cast<const char*>(W), ldw_bytes, epi, row_tiles);
}

template <typename Epi, int XR>
void launch_skinny_kwaves(cigemmContext* ctx, int64_t M, int64_t N, int64_t K, const void* X,
                          int64_t ldx_bytes, const void* W, int64_t ldw_bytes, const Epi& epi) {
  if constexpr (XR == 32) {
    const int cus = ctx->num_cus > 0 ? ctx->num_cus : 256;
    if (N / NK8KW<XR>::BN <= cus) {
      launch_skinny_kwaves_ring<Epi, XR, true>(ctx, M, N, K, X, ldx_bytes, W, ldw_bytes, epi);
      return;
    }
  }
  launch_skinny_kwaves_ring<Epi, XR, false>(ctx, M, N, K, X, ldx_bytes, W, ldw_bytes, epi);
}

// Few slabs and more than 8 rows of x: the rows are cut into tiles of 8 (or 16) and every tile
// gets workgroups of its own, as long as all of them find a compute unit -- a slab's weights
// then cross the fabric once and are read from the XCD's L2 by the other tiles.  One workgroup
// per slab leaves most of the chip idle here and moves as many bytes of x as of W at 32 rows
// (weights rotated, us per call: 4096 x 11008 M = 16 13.9 -> 12.5, M = 32 17.1 -> 13.5;
// 2048 x 8192 M = 32 12.3 -> 8.9 with four tiles of 8, 9.8 with two of 16; with more workgroups
// than units it loses: 5120 x 5120 M = 32 10.3 -> 12.8, 3072 x 8192 in four tiles 12.8 -> 14.4).
// Returns the number of row tiles for tiles of `xr` rows, 0 when that does not apply.
inline int nk8_row_tiles(const cigemmContext* ctx, int64_t M, int64_t N, int xr) {
  return skinny_plan::nk8_row_tiles(M, N, xr, ctx->num_cus);
}

// (A variant with 1024-byte stages, each wave moving 256 contiguous bytes of every weight row --
// 4 rows x 256 bytes per DMA instruction, as the 16-bit kernel's 128-column slabs do -- was built
// and measured for M <= 8: slower, 17.8 against 14.1 us at N = K = 8192, with its ring of four
// 40 KiB stages; level only at K = 28672.  Not kept.)
//
// int8 N x K: the kernel above unless the weights are a few slabs of a very long K (then the
// K ranges of the split-K kernel spread the stream over more compute units).  Measured at
// M = 8, per call: 4096 x 8192 13.2 -> 10.1 us, 4096 x 4096 10.9 -> 7.2, 1024 x 8192 11.1 ->
// 8.7, 128 x 8192 9.2 -> 7.2 (7.2 us is the floor of the test's launch path).
// Returns true when the first one ran.
template <typename Epi>
bool launch_skinny_nk8(cigemmContext* ctx, int64_t M, int64_t N, int64_t K, const void* X,
                       int64_t ldx_bytes, const void* W, int64_t ldw_bytes, const Epi& epi) {
  const int cus = ctx->num_cus > 0 ? ctx->num_cus : 256;
  // (N not a multiple of the split-K kernel's 128-column slabs: only this kernel takes it)
  if (N / 32 >= cus / 4 || K <= 16384 || N % GeoNK8::BN) {
    if (M <= 8)
      launch_skinny_kwaves<Epi, 8>(ctx, M, N, K, X, ldx_bytes, W, ldw_bytes, epi);
    else if (const int t8 = nk8_row_tiles(ctx, M, N, 8))
      launch_skinny_kwaves_row_tiles<Epi, 8>(ctx, M, N, K, X, ldx_bytes, W, ldw_bytes, epi, t8);
    else if (const int t16 = nk8_row_tiles(ctx, M, N, 16))
      launch_skinny_kwaves_row_tiles<Epi, 16>(ctx, M, N, K, X, ldx_bytes, W, ldw_bytes, epi, t16);
    else if (M <= 16)
      launch_skinny_kwaves<Epi, 16>(ctx, M, N, K, X, ldx_bytes, W, ldw_bytes, epi);
    else
      launch_skinny_kwaves<Epi, 32>(ctx, M, N, K, X, ldx_bytes, W, ldw_bytes, epi);
    return true;
  }
  launch_skinny<GeoNK8>(ctx, M, N, K, X, ldx_bytes, W, ldw_bytes, epi);
  return false;
}

// ---- K x N weights, slabs of whole lines: K over the waves ------------------------------------
// The kernel above gives a workgroup 256 columns and a workgroup barrier per stage, and splits K
// over up to 16 workgroups per slab.  Here a workgroup owns a slab of one or two whole 128-byte
// lines of every weight row (64 or 128 columns of a 16-bit type, 128 of int8; half lines stream
// at two thirds of the rate) and a K range; inside it the four waves split k (a stage is 64 rows
// of k -- 128 for int8 --, wave w moves and multiplies rows 16 w .. 16 w + 15 of every stage and
// never touches what another wave moved: no workgroup barrier in the loop), their four partial
// 32-row tiles are summed through LDS in wave order, and only then do K ranges meet: two ranges
// through one atomic exchange per pair of outputs, more through the partial / arrival-counter
// exchange of the kernel above.
// Per wave and stage: the W piece [16 k][slab] (2 or 4 KiB, DMA instructions of 1 KiB of whole
// rows each) and the x piece [XR m][16 k] (XR x 32 bytes of the slot, XR = 8, 16 or 32, the
// smallest that holds M; one DMA instruction of 2 M lanes fills its first M rows), in a ring of
// NSTAGES slots private to the wave.  The rings are short enough for two workgroups to share a
// compute unit's LDS (3 or 4 slots beside 4 KiB W pieces, 6 beside 2 KiB): a launch of more
// workgroups than units then has no second round that waits for the first, and a single
// workgroup on a unit streams no slower than with rings twice as deep (measured, M = 1 / 32, 7
// slots -> 4 / 3: N = K = 8192 26.6 / 29.5 -> 26.1 / 28.4 us, 28672 x 8192 80.4 / 90.7 ->
// 79.8 / 85.1).
template <int EB_, int XR_, int COLS_>
struct KN16KW {
  static constexpr int EB = EB_;                       // bytes per element: 2 (fp16, bf16) or 1 (int8)
  static constexpr int BN = COLS_;                     // 16-bit: 64 or 128 (one or two lines per
                                                       // weight row); int8: 128 (one line)
  static constexpr int KW = 32 / EB;                   // k rows per wave and stage = one MFMA's k
  static constexpr int K_STAGE = 4 * KW;               // k rows per stage and workgroup
  static constexpr int XR = XR_;
  static constexpr int ROW_BYTES = EB * BN;
  static constexpr int W_BYTES = KW * ROW_BYTES;       // per wave and stage
  static constexpr int W_DMAS = W_BYTES / 1024;        // one instruction moves 1 KiB of whole rows
  static constexpr int MT = XR > 32 ? 2 : 1;           // 32-row tiles of x (XR = 64: two)
  static constexpr int X_BYTES = XR * 32;              // 32 bytes of k per row of x
  static constexpr int SLOT_BYTES = W_BYTES + X_BYTES;
  // ring slots per wave: what lets two workgroups share the LDS of a compute unit
  static constexpr int NSTAGES = W_BYTES <= 1024 ? 8 : W_BYTES == 2048 ? 6 : XR <= 16 ? 4 : 3;
  static constexpr int DPS = W_DMAS + MT;              // DMA instructions per wave and stage
  static constexpr int WAVE_BYTES = NSTAGES * SLOT_BYTES;
  static constexpr int RED_LD = BN + 4;                // words per row of the reduction tiles
  static constexpr int RED_BYTES = 4 * 32 * RED_LD * 4;
  static constexpr int LDS_BYTES = 4 * WAVE_BYTES > RED_BYTES ? 4 * WAVE_BYTES : RED_BYTES;
  static constexpr int PART_WORDS = BN / 16;           // 64-bit words per thread and 32-row tile
                                                       // of a partial result
};

template <typename Math, typename Epi, int XR, int COLS>
__global__ __launch_bounds__(256, 2) void skinny_kn16_kwaves_kernel(
    int M, int N, int stages, int splits, const char* __restrict__ X, int64_t ldx,
    const char* __restrict__ W, int64_t ldw, Epi epi, uint64_t* __restrict__ partials,
    uint32_t* __restrict__ counters, uint64_t* __restrict__ swap_words) {
  typedef KN16KW<Math::ELEM_BYTES, XR, COLS> G;
  typedef tile::lds_i16x4 lds_i16x4;
  typedef tile::lds_i32x2 lds_i32x2;
  typedef typename Math::scalar_t scalar_t;           // float, or int32_t for int8
  constexpr int EB = G::EB;
  constexpr int NS = G::NSTAGES, DIST = NS - 1;
  constexpr int NT = COLS / 32;                       // 32-column tiles of the slab
  constexpr int MT = G::MT;                           // 32-row tiles of x
  constexpr int PIECES = G::ROW_BYTES / 16;           // 16-byte pieces of a slab row
  constexpr int ROWS_PER_DMA = 64 / PIECES;
  constexpr int QUADS = COLS / 32;                    // groups of 4 columns per thread of the reduction
  extern __shared__ __attribute__((aligned(1024))) char lds[];
  __shared__ int is_last;
  const int t = threadIdx.x, l = t & 63;
  const int w = __builtin_amdgcn_readfirstlane(t >> 6);
  const int slab = blockIdx.x / splits, split = blockIdx.x % splits;
  const int64_t n0 = (int64_t)slab * G::BN;
  // K range `split` of `splits`: stages [split * stages / splits, (split + 1) * stages / splits),
  // as even as the stage count allows; this wave's k rows of its first stage
  // (32-bit: split < 16 and stages < 2^25, and a 64-bit division costs a few hundred cycles)
  const int s_begin = (int)((unsigned)(split * stages) / (unsigned)splits);
  const int KTS = (int)((unsigned)((split + 1) * stages) / (unsigned)splits) - s_begin;
  const int64_t k0 = (int64_t)s_begin * G::K_STAGE + G::KW * w;
  char* const wave_lds = lds + w * G::WAVE_BYTES;
  const uint32_t wave_base =
      (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)lds + w * G::WAVE_BYTES;

  // lane l of a W instruction: row l / PIECES of its rows, 16-byte piece l % PIECES of the row;
  // of the x instruction: row l / 2, piece l % 2, lanes of rows below M only (the rows of the
  // slot past M keep whatever the LDS held: an output row depends on its own row of x alone, and
  // rows >= M are never stored)
  const char* w_src = W + (k0 + l / PIECES) * ldw + n0 * EB + ((l % PIECES) << 4);
  const char* x_src = X + (int64_t)(l >> 1) * ldx + k0 * EB + ((l & 1) << 4);
  auto issue = [&](int st, int slot) {
    const uint32_t dst = wave_base + slot * G::SLOT_BYTES;
    const char* ws = w_src + (int64_t)st * G::K_STAGE * ldw;
#pragma unroll
    for (int i = 0; i < G::W_DMAS; ++i) dma16(ws + (int64_t)(ROWS_PER_DMA * i) * ldw, dst + 1024 * i);
    if (l < 2 * M) dma16(x_src + st * (G::K_STAGE * EB), dst + G::W_BYTES);
    // rows 32 and up (the launcher picks XR = 64 only for M > 32: lane 0 always takes part, so
    // the instruction is issued and counted every time)
    if constexpr (MT == 2)
      if (l + 64 < 2 * M) dma16(x_src + 32 * ldx + st * (G::K_STAGE * EB), dst + G::W_BYTES + 1024);
  };

  typename Math::acc_t acc[MT][NT];
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int j = 0; j < NT; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0;
#pragma unroll
  for (int st = 0; st < DIST; ++st)
    if (st < KTS) issue(st, st);

  // fragment addresses within a slot: the transposing read of the W piece (16-bit: within 16
  // lanes, lane i supplies 8 bytes of row i / 4 and receives the 4 k-values of column i, lanes
  // 32-63 take rows 8-15, a second read the rows 4 further on; bytes: row i / 2, 8 k-values,
  // lanes 32-63 rows 16-31, the second read the rows 8 further on), and 16 bytes of row
  // l % XR of the x piece
  const int w_off = EB == 2 ? (8 * (l >> 5) + ((l & 15) >> 2)) * G::ROW_BYTES +
                                  (16 * ((l >> 4) & 1) + 4 * (l & 3)) * 2
                            : (16 * (l >> 5) + ((l & 15) >> 1)) * G::ROW_BYTES +
                                  16 * ((l >> 4) & 1) + 8 * (l & 1);
  const int x_off = G::W_BYTES + (l & ((XR < 32 ? XR : 32) - 1)) * 32 + ((l >> 5) << 4);
  int slot = 0, dma_slot = DIST;
  for (int s = 0; s < KTS; ++s) {
    // Stage s landed for this wave; nothing is fetched past the K range, so fewer stages are
    // in flight at its end.  The slot refilled now is the one of stage s - 1, whose fragments
    // this wave's own MFMAs have consumed.
    wait_stages_in_flight<G::DPS, DIST - 1>(KTS - 1 - s < DIST - 1 ? KTS - 1 - s : DIST - 1);
    __builtin_amdgcn_sched_barrier(0);
    if (s + DIST < KTS) issue(s + DIST, dma_slot);
    const char* sl = wave_lds + slot * G::SLOT_BYTES;
    u32x4 xf[MT];
#pragma unroll
    for (int i = 0; i < MT; ++i) xf[i] = *reinterpret_cast<const u32x4*>(sl + x_off + 1024 * i);
#pragma unroll
    for (int j = 0; j < NT; ++j) {
      u32x4 wf;
      if constexpr (EB == 2) {
        const i16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4*)(sl + w_off + 64 * j));
        const i16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
            (lds_i16x4*)(sl + w_off + 64 * j + 4 * G::ROW_BYTES));
        wf = __builtin_shufflevector(__builtin_bit_cast(u32x2, lo), __builtin_bit_cast(u32x2, hi),
                                     0, 1, 2, 3);
      } else {
        const i32x2 lo = __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_i32x2*)(sl + w_off + 32 * j));
        const i32x2 hi = __builtin_amdgcn_ds_read_tr8_b64_v2i32(
            (lds_i32x2*)(sl + w_off + 32 * j + 8 * G::ROW_BYTES));
        wf = __builtin_shufflevector(__builtin_bit_cast(u32x2, lo), __builtin_bit_cast(u32x2, hi),
                                     0, 1, 2, 3);
      }
#pragma unroll
      for (int i = 0; i < MT; ++i) acc[i][j] = Math::mfma(wf, xf[i], acc[i][j]);
    }
    slot = slot + 1 == NS ? 0 : slot + 1;
    dma_slot = dma_slot + 1 == NS ? 0 : dma_slot + 1;
  }
  __syncthreads();  // every wave done with its ring (nothing is in flight): reuse it

  // acc[i][j][4 q + e] = this wave's part of y[32 i + l % 32][n0 + 32 j + 8 q + 4 (l / 32) + e].
  // One 32-row tile of x at a time goes through the reduction tiles: thread t takes row t / 8
  // (+ 32 i), columns 4 QUADS (t % 8) .. + 4 QUADS - 1, summed over the waves in wave order.
  scalar_t* red = reinterpret_cast<scalar_t*>(lds);  // [4 waves][32 m][RED_LD]
  const int m0 = t >> 3, c = (t & 7) * 4 * QUADS;
  scalar_t sums[MT][4 * QUADS];
#pragma unroll
  for (int i = 0; i < MT; ++i) {
    if (i > 0) __syncthreads();  // the tiles of the rows before are read
#pragma unroll
    for (int j = 0; j < NT; ++j)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        scalar_t* dst = red + (w * 32 + (l & 31)) * G::RED_LD + 32 * j + 8 * q + 4 * (l >> 5);
        const u32x4 v = {__builtin_bit_cast(uint32_t, (scalar_t)acc[i][j][4 * q]),
                         __builtin_bit_cast(uint32_t, (scalar_t)acc[i][j][4 * q + 1]),
                         __builtin_bit_cast(uint32_t, (scalar_t)acc[i][j][4 * q + 2]),
                         __builtin_bit_cast(uint32_t, (scalar_t)acc[i][j][4 * q + 3])};
        *reinterpret_cast<u32x4*>(dst) = v;
      }
    __syncthreads();
#pragma unroll
    for (int h = 0; h < QUADS; ++h) {
#pragma unroll
      for (int ww = 0; ww < 4; ++ww) {
        const u32x4 p =
            *reinterpret_cast<const u32x4*>(red + (ww * 32 + m0) * G::RED_LD + c + 4 * h);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const uint32_t bits = p[e];
          const scalar_t v = __builtin_bit_cast(scalar_t, bits);
          sums[i][4 * h + e] = ww == 0 ? v : sums[i][4 * h + e] + v;
        }
      }
    }
  }
  if (splits == 1) {
#pragma unroll
    for (int i = 0; i < MT; ++i) {
      const int m = m0 + 32 * i;
      if (m < M) {
#pragma unroll
        for (int h = 0; h < QUADS; ++h)
          epi(m, n0 + c + 4 * h, sums[i][4 * h], sums[i][4 * h + 1], sums[i][4 * h + 2],
              sums[i][4 * h + 3]);
      }
    }
    return;
  }
  // ---- two K ranges meet through one atomic exchange per 64-bit word.  The word of (slab,
  // word, thread) is zero between calls; each of the two workgroups swaps its pair of partial
  // sums in.  The one that gets zero back was first and is done: its pair now waits in the
  // word.  The one that gets a pair back has both, writes the two outputs and puts the zero
  // back.  The data travels inside the atomic operation itself, so nothing else has to be
  // ordered: no partial tile in memory, no counter, no wait, one trip to the coherence point
  // instead of three.  Which workgroup finishes a word may differ from word to word; a + b is
  // the same bits either way, and the sum is formed as (0 + range 0) + range 1 like the
  // reduction below.  A pair of two +0.0f would look like the empty word: it travels as two
  // -0.0f, which 0 + x turns back into +0.0f.
  if constexpr (EB == 2) {
  if (splits == 2 && swap_words) {
#pragma unroll
    for (int i = 0; i < MT; ++i) {
      const int m = m0 + 32 * i;
      const scalar_t* sum = sums[i];
      if (m < M) {
        uint64_t* word = swap_words + ((int64_t)(slab * MT + i) * G::PART_WORDS) * 256 + t;
        uint64_t got[2 * QUADS];
#pragma unroll
        for (int p = 0; p < 2 * QUADS; ++p) {
          uint64_t mine = (uint64_t)__builtin_bit_cast(uint32_t, sum[2 * p]) |
                          ((uint64_t)__builtin_bit_cast(uint32_t, sum[2 * p + 1]) << 32);
          if (mine == 0) mine = 0x8000000080000000ull;
          got[p] = __hip_atomic_exchange(word + 256 * p, mine, __ATOMIC_RELAXED,
                                         __HIP_MEMORY_SCOPE_AGENT);
        }
#pragma unroll
        for (int p = 0; p < 2 * QUADS; ++p) {
          if (got[p] == 0) continue;
          const float o0 = __builtin_bit_cast(float, (uint32_t)got[p]);
          const float o1 = __builtin_bit_cast(float, (uint32_t)(got[p] >> 32));
          const float a0 = split == 0 ? sum[2 * p] : o0, b0 = split == 0 ? o0 : sum[2 * p];
          const float a1 = split == 0 ? sum[2 * p + 1] : o1,
                      b1 = split == 0 ? o1 : sum[2 * p + 1];
          epi.pair(m, n0 + c + 2 * p, (0.0f + a0) + b0, (0.0f + a1) + b1);
          __hip_atomic_store(word + 256 * p, (uint64_t)0, __ATOMIC_RELAXED,
                             __HIP_MEMORY_SCOPE_AGENT);
        }
      }
    }
    return;
  }
  }
  // ---- more K ranges: same exchange as in skinny_kernel (partials as agent-scope 64-bit words,
  // laid out [split][slab][tile of x][word][thread]; the last workgroup of the slab sums in split
  // order)
  const int slabs = gridDim.x / splits;
  auto part = [&](int sp, int i) {
    return partials + ((int64_t)((sp * slabs + slab) * MT + i) * G::PART_WORDS) * 256 + t;
  };
#pragma unroll
  for (int i = 0; i < MT; ++i)
    if (m0 + 32 * i < M) {
      uint64_t* dst = part(split, i);
#pragma unroll
      for (int h = 0; h < QUADS; ++h)
        store_partial(dst + 512 * h, sums[i][4 * h], sums[i][4 * h + 1], sums[i][4 * h + 2],
                      sums[i][4 * h + 3]);
    }
  __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): this lane's partial stores are acknowledged
  __syncthreads();
  if (t == 0) {
    const uint32_t old = __hip_atomic_fetch_add(counters + slab, 1u, __ATOMIC_RELAXED,
                                                __HIP_MEMORY_SCOPE_AGENT);
    is_last = old == (uint32_t)(splits - 1);
  }
  __syncthreads();
  if (!is_last) return;
#pragma unroll
  for (int i = 0; i < MT; ++i) {
    const int m = m0 + 32 * i;
    if (m < M) {
      scalar_t q4[QUADS][4];
      const int64_t stride = (int64_t)slabs * MT * G::PART_WORDS * 256;
      sum_partials_n<scalar_t, QUADS>(part(0, i), stride, splits, q4);
#pragma unroll
      for (int h = 0; h < QUADS; ++h)
        epi(m, n0 + c + 4 * h, q4[h][0], q4[h][1], q4[h][2], q4[h][3]);
    }
  }
  if (t == 0) __hip_atomic_store(counters + slab, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// K ranges per slab for the kernel above: skinny_plan.h has the rule.
inline int kn16_kwaves_splits(const cigemmContext* ctx, int64_t N, int64_t kts, int cols,
                              int x_tiles) {
  return skinny_plan::kwaves_splits(N / cols, kts, cols, ctx->num_cus, ctx->ws_counter_bytes,
                                    ctx->ws_partial_bytes / x_tiles);
}

template <typename Math, typename Epi, int XR, int COLS>
void launch_kn16_kwaves_xr(cigemmContext* ctx, int64_t M, int64_t N, int64_t K, const void* X,
                           int64_t ldx_bytes, const void* W, int64_t ldw_bytes, const Epi& epi) {
  typedef KN16KW<Math::ELEM_BYTES, XR, COLS> G;
  static_assert(2 * (G::LDS_BYTES + 64) <= 160 * 1024,
                "rings and arrival flags of two workgroups must fit the LDS");
  auto kern = skinny_kn16_kwaves_kernel<Math, Epi, XR, COLS>;
  static std::atomic<uint64_t> lds_set{0};
  if (!ensure_dynamic_lds(ctx, (const void*)kern, G::LDS_BYTES, lds_set)) return;
  const int64_t kts = K / G::K_STAGE;
  const int splits = kn16_kwaves_splits(ctx, N, kts, COLS, G::MT);
  hipLaunchKernelGGL(kern, dim3((unsigned)(N / G::BN * splits)), dim3(256), G::LDS_BYTES,
                     ctx->stream, (int)M, (int)N, (int)kts, splits,
                     static_cast<const char*>(X), ldx_bytes, static_cast<const char*>(W),
                     ldw_bytes, epi, static_cast<uint64_t*>(ctx->workspace),
                     reinterpret_cast<uint32_t*>(static_cast<char*>(ctx->workspace) +
                                                 ctx->ws_partial_bytes),
                     // one exchange word per pair of columns and row of x: 128 bytes per column
                     // and 32-row tile
                     (size_t)N * 128 * G::MT <= ctx->ws_swap_bytes
                         ? reinterpret_cast<uint64_t*>(static_cast<char*>(ctx->workspace) +
                                                       ctx->ws_partial_bytes +
                                                       ctx->ws_counter_bytes)
                         : nullptr);
}

// Slab widths of the 16-bit types: 64 columns (one line per weight row) and 128 (two lines);
// kn16_choice says which.  Half a line per row (32-column slabs: 256 slabs at N = 8192, no
// exchange between workgroups at all) streams at two thirds of the rate: 45 against 30 us at
// N = K = 8192, 47 against 28 at 16384 x 4096, level only at N = 1024.  int8 K x N weights use
// 128 columns (one line); 256 columns were measured slower there (8192 x 8192: 17.8 -> 19.2 us).
template <typename Math, int COLS, typename Epi>
void launch_kn16_kwaves(cigemmContext* ctx, int64_t M, int64_t N, int64_t K, const void* X,
                        int64_t ldx_bytes, const void* W, int64_t ldw_bytes, const Epi& epi) {
  if (M <= 8)
    launch_kn16_kwaves_xr<Math, Epi, 8, COLS>(ctx, M, N, K, X, ldx_bytes, W, ldw_bytes, epi);
  else if (M <= 16)
    launch_kn16_kwaves_xr<Math, Epi, 16, COLS>(ctx, M, N, K, X, ldx_bytes, W, ldw_bytes, epi);
  else if (M <= 32)
    launch_kn16_kwaves_xr<Math, Epi, 32, COLS>(ctx, M, N, K, X, ldx_bytes, W, ldw_bytes, epi);
  else if constexpr (COLS == 128)  // two tiles of x: the rings only fit beside 4 KiB W pieces
    launch_kn16_kwaves_xr<Math, Epi, 64, COLS>(ctx, M, N, K, X, ldx_bytes, W, ldw_bytes, epi);
}

template <typename Geo>
bool skinny_shape_ok(const cigemmContext* ctx, int64_t M, int64_t N, int64_t K, int elem,
                     const void* X, int64_t ldx, const void* W, int64_t ldw,
                     int64_t max_m = XROWS) {
  if (!ctx->workspace) return false;
  if (M < 1 || M > max_m || N <= 0 || K <= 0) return false;
  if (N % Geo::BN || K % Geo::K_ELEMS) return false;
  if ((ldx * elem) % 16 || (ldw * elem) % 16) return false;
  if (((uintptr_t)X & 15) || ((uintptr_t)W & 15)) return false;
  if (N / Geo::BN * 16 > 2147483647LL || N > 2147483647LL) return false;
  return true;
}

// the shape conditions of the int8 kernel without split-K: 32-column slabs, 128-k chunks
struct Slab32 {
  static constexpr int BN = 32, K_ELEMS = 128;
};

// 33 to 64 rows of x (two 32-row tiles per wave, x pieces half the size of the W pieces): the
// K-over-the-waves kernel beats the tile kernel's 64-row tiles with split-K and a reduction launch
// when its slabs x ranges put exactly one workgroup on every compute unit (M = 33 / 64, weights
// rotated: N = K = 4096 14.5 / 16.1 against 17.5 / 19.3 us, N = K = 8192 30.0 / 33.4 against 35.0 /
// 36.9, 32768 x 2048 26.3 / 28.0 against 30.0 / 31.5, 4096 x 11008 24.3 / 27.1 against 26.6 /
// 29.5; int8 K x N 16384 x 4096 19.7 / 22.6 against 22.2 / 24.4), and loses where it does not
// (11008 x 4096, 430 workgroups: 25.9 / 32.4 against 22.4 / 24.0; 28672 x 8192, 224: 85.3 /
// 105.4 against 81.5 / 85.3; 13824 x 5120, 216: 32.4 / 40.2 against 29.8 / 32.5): the tile
// kernel's smaller workgroups spread more evenly.  Forcing the family takes every shape.
inline bool two_tiles_pay(const cigemmContext* ctx, int64_t slabs, int64_t kts, int cols) {
  if (ctx->algo == CIGEMM_ALGO_SKINNY) return true;
  return skinny_plan::two_tiles_fit(slabs, kts, cols, ctx->num_cus, ctx->ws_counter_bytes,
                                    ctx->ws_partial_bytes);
}

// Which 16-bit decode kernel.  The K-over-the-waves kernel takes every shape it can (N and K
// multiples of 64); the 256-column kernel with a barrier per stage is left with K a multiple of
// 32 but not of 64 (with N a multiple of 256), where it is the only one: everywhere else it is
// slower, up to twice with more than 16 rows of x (N = 8192, K = 1024, M = 32: 14.1 against
// 7.2 us; N = K = 4096: 19.4 against 10.7 at M = 1).
// Slab width: large weight matrices take 128-column slabs -- two lines, 256 contiguous bytes,
// per weight row and DMA row -- which stream faster and re-read x half as often (M = 1 / 32:
// N = K = 8192 28.4 / 32.0 -> 26.0 / 28.4 us, 28672 x 8192 95.9 / 127.4 -> 79.4 / 84.6, 22016 x
// 4096 44.3 / 59.1 -> 34.1 / 38.9, 6144 x 6144 18.0 / 22.4 -> 17.3 / 19.2), at the price of half
// as many slabs, so twice the K ranges to exchange: no faster up to 4096 x 4096 weights (level
// there and at 8192 x 2048; 4096 x 2048: 7.8 / 8.5 against 8.0 / 9.6), slower below 32 slabs or
// 2048 k (2048 x 8192: 11.1 / 12.4 against 13.0 / 15.8 us, 8192 x 1024: 7.1 / 7.3 against 7.4 /
// 8.8).
// 0: neither, 1: 64-column slabs, 2: 256-column slabs with a barrier per stage, 3: 128-column slabs.
inline int kn16_choice(const cigemmContext* ctx, int64_t M, int64_t N, int64_t K) {
  const bool kw_ok = N % 64 == 0 && K % 64 == 0 && (size_t)(N / 64) * 4 <= ctx->ws_counter_bytes;
  const bool sk_ok = N % GeoKN16<tile::MathBF16>::BN == 0 && K % GeoKN16<tile::MathBF16>::K_ELEMS == 0;
  if (M > XROWS)  // 33 to 64 rows of x: two tiles, 128-column slabs only
    return kw_ok && N % 128 == 0 && N / 128 >= 32 && K >= 2048 &&
                   two_tiles_pay(ctx, N / 128, K / 64, 128)
               ? 3
               : 0;
  if (kw_ok && N % 128 == 0 && N / 128 >= 32 && K >= 2048 && N * K > (int64_t)4096 * 4096)
    return 3;
  if (kw_ok) return 1;
  return sk_ok ? 2 : 0;
}

// Policy + launch of the 16-bit decode GEMM on a context whose workspace is in place (a handle's,
// or the static array of the entry point that allocates nothing): both must make the same
// choices so that they give the same bits.  Returns the kernel's name, null when neither kernel
// takes the shape (nothing was launched).
template <typename Math, typename E16>
const char* launch_skinny_16_on(cigemmContext* ctx, int64_t M, int64_t N, int64_t K,
                                const uint16_t* A, int64_t lda, const uint16_t* B, int64_t ldb,
                                uint16_t* C, int64_t ldc, bool bf16) {
  const int which = kn16_choice(ctx, M, N, K);
  if (which == 3) {
    launch_kn16_kwaves<Math, 128>(ctx, M, N, K, A, lda * 2, B, ldb * 2, EpiStore16x4<E16>{C, ldc});
    if (M > XROWS) return bf16 ? "bf16_skinny_64x128_kwaves" : "f16_skinny_64x128_kwaves";
    return bf16 ? "bf16_skinny_32x128_kwaves" : "f16_skinny_32x128_kwaves";
  }
  if (which == 1) {
    launch_kn16_kwaves<Math, 64>(ctx, M, N, K, A, lda * 2, B, ldb * 2, EpiStore16x4<E16>{C, ldc});
    return bf16 ? "bf16_skinny_32x64_kwaves" : "f16_skinny_32x64_kwaves";
  }
  if (which == 0) return nullptr;
  launch_skinny<GeoKN16<Math>>(ctx, M, N, K, A, lda * 2, B, ldb * 2, EpiStore16x4<E16>{C, ldc});
  return bf16 ? "bf16_skinny_32x256_ring8" : "f16_skinny_32x256_ring8";
}

}  // namespace

// the alignment conditions common to both 16-bit kernels; kn16_choice has the shape conditions
struct Slab16Any {
  static constexpr int BN = 64, K_ELEMS = 32;
};

bool launch_skinny_16(cigemmContext* ctx, bool bf16, int64_t M, int64_t N, int64_t K,
                      const uint16_t* A, int64_t lda, const uint16_t* B, int64_t ldb, uint16_t* C,
                      int64_t ldc) {
  if (!skinny_shape_ok<Slab16Any>(ctx, M, N, K, 2, A, lda, B, ldb, 2 * XROWS)) return false;
  if (ldc % 4 || ((uintptr_t)C & 7)) return false;
  const char* name =
      bf16 ? launch_skinny_16_on<tile::MathBF16, BF16>(ctx, M, N, K, A, lda, B, ldb, C, ldc, true)
           : launch_skinny_16_on<tile::MathF16, F16>(ctx, M, N, K, A, lda, B, ldb, C, ldc, false);
  if (!name) return false;
  ctx->last_kernel = name;
  return true;
}

// int8 K x N weights: the K-over-the-waves kernel of the 16-bit types with 128-column slabs (one
// 128-byte line per weight row) and 128 k per stage; N and K multiples of 128.  Other shapes go
// to the tile kernel (64-row tiles, split-K).
struct SlabKN8 {
  static constexpr int BN = 128, K_ELEMS = 128;
};
static bool launch_skinny_i8_kn(cigemmContext* ctx, int64_t M, int64_t N, int64_t K,
                                const int8_t* A, int64_t lda, const int8_t* B, int64_t ldb,
                                int32_t* C, int64_t ldc, const DequantArgs* dq) {
  if (!skinny_shape_ok<SlabKN8>(ctx, M, N, K, 1, A, lda, B, ldb, 2 * XROWS)) return false;
  if (M > XROWS && !two_tiles_pay(ctx, N / SlabKN8::BN, K / SlabKN8::K_ELEMS, SlabKN8::BN))
    return false;
  if ((size_t)(N / SlabKN8::BN) * 4 > ctx->ws_counter_bytes) return false;
  if (!dq) {
    if (ldc % 4 || ((uintptr_t)C & 15)) return false;
    launch_kn16_kwaves<tile::MathI8, 128>(ctx, M, N, K, A, lda, B, ldb, EpiStoreI32x4{C, ldc});
    ctx->last_kernel = M > XROWS ? "i8_skinny_64x128_kwaves_kn" : "i8_skinny_32x128_kwaves_kn";
    return true;
  }
  if (dq->out_bf16 ? (dq->ldo % 4 || ((uintptr_t)dq->out & 7))
                   : (dq->ldo % 4 || ((uintptr_t)dq->out & 15)))
    return false;
  if (dq->sb_vec && ((uintptr_t)dq->sb & 15)) return false;
  if (dq->acc_out && (dq->ldacc % 4 || ((uintptr_t)dq->acc_out & 15))) return false;
#define CIG_DQ(OB, DA)                                                                          \
  launch_kn16_kwaves<tile::MathI8, 128>(ctx, M, N, K, A, lda, B, ldb,                            \
                                        EpiDequantX4<OB, DA>{dq->out, dq->ldo, dq->sa, dq->sb,   \
                                                             dq->sa_vec, dq->sb_vec,             \
                                                             dq->acc_out, dq->ldacc})
  const bool dump = dq->acc_out != nullptr;
  if (dq->out_bf16) {
    if (dump) CIG_DQ(true, true); else CIG_DQ(true, false);
  } else {
    if (dump) CIG_DQ(false, true); else CIG_DQ(false, false);
  }
#undef CIG_DQ
  ctx->last_kernel =
      M > XROWS ? "i8_skinny_64x128_kwaves_kn_dequant" : "i8_skinny_32x128_kwaves_kn_dequant";
  return true;
}

bool launch_skinny_i8(cigemmContext* ctx, int64_t M, int64_t N, int64_t K, const int8_t* A,
                      int64_t lda, const int8_t* B, int64_t ldb, bool b_nk, int32_t* C,
                      int64_t ldc, const DequantArgs* dq) {
  if (!b_nk) return launch_skinny_i8_kn(ctx, M, N, K, A, lda, B, ldb, C, ldc, dq);
  if (!skinny_shape_ok<Slab32>(ctx, M, N, K, 1, A, lda, B, ldb)) return false;
  if (!dq) {
    if (ldc % 4 || ((uintptr_t)C & 15)) return false;
    const bool kw = launch_skinny_nk8(ctx, M, N, K, A, lda, B, ldb, EpiStoreI32x4{C, ldc});
    ctx->last_kernel = kw ? "i8_skinny_32x32_kwaves_nk" : "i8_skinny_32x128_ring7_nk";
    return true;
  }
  if (dq->out_bf16 ? (dq->ldo % 4 || ((uintptr_t)dq->out & 7))
                   : (dq->ldo % 4 || ((uintptr_t)dq->out & 15)))
    return false;
  if (dq->sb_vec && ((uintptr_t)dq->sb & 15)) return false;
  if (dq->acc_out && (dq->ldacc % 4 || ((uintptr_t)dq->acc_out & 15))) return false;
#define CIG_DQ(OB, DA)                                                                          \
  launch_skinny_nk8(ctx, M, N, K, A, lda, B, ldb,                                               \
                    EpiDequantX4<OB, DA>{dq->out, dq->ldo, dq->sa, dq->sb, dq->sa_vec,          \
                                         dq->sb_vec, dq->acc_out, dq->ldacc})
  const bool dump = dq->acc_out != nullptr;
  bool kw;
  if (dq->out_bf16) {
    kw = dump ? CIG_DQ(true, true) : CIG_DQ(true, false);
  } else {
    kw = dump ? CIG_DQ(false, true) : CIG_DQ(false, false);
  }
#undef CIG_DQ
  ctx->last_kernel = kw ? "i8_skinny_32x32_kwaves_nk_dequant" : "i8_skinny_32x128_ring7_nk_dequant";
  return true;
}

// ---- the entry point that allocates nothing --------------------------------------------------
// For callers that cannot allocate device memory (code under HIP graph capture, tight serving
// loops, harnesses that forbid it): the bf16 decode GEMM above with its split-K partials and
// arrival counters in a file-scope device array instead of a handle's workspace, and no handle
// (creating one allocates).  Each GPU the library runs on holds the array until the process
// ends.  Every call on a GPU shares that GPU's array: calls that overlap on one GPU race.
namespace {

constexpr size_t kStaticPartialBytes = (size_t)16 << 20;  // covers every N <= kStaticMaxN
constexpr size_t kStaticCounterBytes = 4096;
constexpr int64_t kStaticMaxN = 16384;
constexpr size_t kStaticSwapBytes = (size_t)kStaticMaxN * 128;  // exchange words of two K ranges
constexpr int kStaticMaxDevices = 64;

static __device__ __align__(256) unsigned char
    scratch[kStaticPartialBytes + kStaticCounterBytes + kStaticSwapBytes];

// `scratch` in host code is only a handle for the runtime's symbol table, not a device
// address: the address of each device's copy is looked up once, with that device current.
struct StaticDevice {
  std::atomic<int> state{0};  // 0 = not looked up, 1 = ready, -1 = unusable (see status)
  cigemmStatus_t status = CIGEMM_STATUS_SUCCESS;
  char* ptr = nullptr;
  int num_cus = 0;
};
StaticDevice g_static_dev[kStaticMaxDevices];
std::mutex g_static_mutex;

cigemmStatus_t static_device_setup(int dev, StaticDevice** out) {
  StaticDevice& d = g_static_dev[dev];
  if (d.state.load(std::memory_order_acquire) == 0) {
    std::lock_guard<std::mutex> lock(g_static_mutex);
    if (d.state.load(std::memory_order_relaxed) == 0) {
      hipDeviceProp_t prop;
      void* p = nullptr;
      if (hipGetDeviceProperties(&prop, dev) != hipSuccess) {
        (void)hipGetLastError();
        d.status = CIGEMM_STATUS_NOT_INITIALIZED;
      } else if (strncmp(prop.gcnArchName, "gfx950", 6) != 0) {
        d.status = CIGEMM_STATUS_ARCH_MISMATCH;
      } else if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) {
        (void)hipGetLastError();
        d.status = CIGEMM_STATUS_INTERNAL_ERROR;
      } else {
        d.ptr = static_cast<char*>(p);
        d.num_cus = prop.multiProcessorCount;
      }
      d.state.store(d.status == CIGEMM_STATUS_SUCCESS ? 1 : -1, std::memory_order_release);
    }
  }
  *out = &d;
  return d.status;
}

// The arrival counters must be zero when the GEMM kernel starts.  A kernel, not a memset: this
// call may be recorded into a graph.
__global__ void clear_counters_kernel(uint32_t* counters, int n, uint64_t* swap_words,
                                      int64_t n_swap_words) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) counters[i] = 0;
  for (int64_t j = i; j < n_swap_words; j += (int64_t)gridDim.x * blockDim.x) swap_words[j] = 0;
}

}  // namespace

void clear_workspace(cigemmContext* ctx) {
  ctx->ws_dirty = 0;
  if (!ctx->workspace) return;
  char* base = static_cast<char*>(ctx->workspace) + ctx->ws_partial_bytes;
  const int counters = (int)(ctx->ws_counter_bytes / 4);
  const int64_t words = (int64_t)(ctx->ws_swap_bytes / 8);
  const int blocks = 4 * (ctx->num_cus > 0 ? ctx->num_cus : 256);
  const int need = (counters + 255) / 256;
  hipLaunchKernelGGL(clear_counters_kernel, dim3(blocks > need ? blocks : need), dim3(256), 0,
                     ctx->stream, reinterpret_cast<uint32_t*>(base), counters,
                     reinterpret_cast<uint64_t*>(base + ctx->ws_counter_bytes), words);
}

namespace {

cigemmStatus_t static_fail(char* err, size_t err_len, cigemmStatus_t st, const char* fmt, ...)
    __attribute__((format(printf, 4, 5)));
cigemmStatus_t static_fail(char* err, size_t err_len, cigemmStatus_t st, const char* fmt, ...) {
  if (err && err_len) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(err, err_len, fmt, ap);
    va_end(ap);
  }
  return st;
}

}  // namespace
}  // namespace cig

extern "C" cigemmStatus_t cigemm_gemm_bf16_static(void* stream, int64_t M, int64_t N, int64_t K,
                                                  const uint16_t* A, int64_t lda,
                                                  const uint16_t* B, int64_t ldb, uint16_t* C,
                                                  int64_t ldc, char* err, size_t err_len) {
  using namespace cig;
  const char* name = "cigemm_gemm_bf16_static";
  if (err && err_len) err[0] = '\0';
  if (M < 0 || N < 0 || K < 0)
    return static_fail(err, err_len, CIGEMM_STATUS_INVALID_VALUE,
                       "%s: negative dimension (M=%lld N=%lld K=%lld)", name, (long long)M,
                       (long long)N, (long long)K);
  if (M == 0 || N == 0) return CIGEMM_STATUS_SUCCESS;
  if (!A || !B || !C)
    return static_fail(err, err_len, CIGEMM_STATUS_INVALID_VALUE, "%s: null pointer", name);
  if (lda < K || ldb < N || ldc < N)
    return static_fail(err, err_len, CIGEMM_STATUS_INVALID_VALUE,
                       "%s: leading dimension too small (lda=%lld ldb=%lld ldc=%lld)", name,
                       (long long)lda, (long long)ldb, (long long)ldc);
  if (M > XROWS || N > kStaticMaxN)
    return static_fail(err, err_len, CIGEMM_STATUS_NOT_SUPPORTED,
                       "%s: M=%lld N=%lld beyond the maximum of this entry point (M <= %d, "
                       "N <= %lld: its scratch memory is a fixed %zu-byte device array)",
                       name, (long long)M, (long long)N, XROWS, (long long)kStaticMaxN,
                       kStaticPartialBytes + kStaticCounterBytes + kStaticSwapBytes);
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) {
    (void)hipGetLastError();
    return static_fail(err, err_len, CIGEMM_STATUS_NOT_INITIALIZED, "%s: no HIP device", name);
  }
  if (dev < 0 || dev >= kStaticMaxDevices)
    return static_fail(err, err_len, CIGEMM_STATUS_NOT_SUPPORTED, "%s: device %d >= %d", name,
                       dev, kStaticMaxDevices);
  StaticDevice* sd = nullptr;
  const cigemmStatus_t st = static_device_setup(dev, &sd);
  if (st != CIGEMM_STATUS_SUCCESS)
    return static_fail(err, err_len, st, "%s: device %d cannot be used (%s)", name, dev,
                       cigemmGetStatusString(st));

  // a context on the stack, with the device array in the place of a handle's workspace
  cigemmContext ctx{};
  ctx.magic = kCtxMagic;
  ctx.device = dev;
  ctx.num_cus = sd->num_cus;
  ctx.stream = static_cast<hipStream_t>(stream);
  ctx.last_kernel = "";
  ctx.algo = CIGEMM_ALGO_SKINNY;
  ctx.workspace = sd->ptr;
  ctx.ws_partial_bytes = kStaticPartialBytes;
  ctx.ws_counter_bytes = kStaticCounterBytes;
  ctx.ws_swap_bytes = kStaticSwapBytes;
  typedef GeoKN16<tile::MathBF16> GB;
  if (!skinny_shape_ok<GB>(&ctx, M, N, K, 2, A, lda, B, ldb) || ldc % 4 || ((uintptr_t)C & 7))
    return static_fail(err, err_len, CIGEMM_STATUS_NOT_SUPPORTED,
                       "%s: needs N %% 256 == 0, K %% 32 == 0, lda and ldb multiples of 8, ldc of "
                       "4, A and B 16-byte and C 8-byte aligned (M=%lld N=%lld K=%lld)",
                       name, (long long)M, (long long)N, (long long)K);
  {
    // every arrival counter either kernel may use (one per 64-column slab at most) and the
    // exchange words of two K ranges (128 bytes per column)
    const int slabs = (int)((N + 63) / 64);
    const int64_t words = (int64_t)slabs * 64 * 16;
    const int blocks = (int)((words / 4 + 255) / 256) > (slabs + 255) / 256
                           ? (int)((words / 4 + 255) / 256) : (slabs + 255) / 256;
    hipLaunchKernelGGL(clear_counters_kernel, dim3(blocks), dim3(256), 0, ctx.stream,
                       reinterpret_cast<uint32_t*>(sd->ptr + kStaticPartialBytes), slabs,
                       reinterpret_cast<uint64_t*>(sd->ptr + kStaticPartialBytes +
                                                   kStaticCounterBytes),
                       words);
  }
  (void)launch_skinny_16_on<tile::MathBF16, BF16>(&ctx, M, N, K, A, lda, B, ldb, C, ldc, true);
  if (ctx.pending_error[0]) {
    (void)hipGetLastError();
    return static_fail(err, err_len, CIGEMM_STATUS_INTERNAL_ERROR, "%s: %s", name,
                       ctx.pending_error);
  }
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess)
    return static_fail(err, err_len, CIGEMM_STATUS_EXECUTION_FAILED, "%s: HIP error: %s", name,
                       hipGetErrorString(e));
  return CIGEMM_STATUS_SUCCESS;
}
