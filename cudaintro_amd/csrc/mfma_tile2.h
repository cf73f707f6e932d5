// The LDS-tiled MFMA GEMM kernel in its two-workgroups-per-compute-unit form.
//
// mfma_tile_kernel (mfma_tile.h) keeps one workgroup per compute unit: while that workgroup
// fills its pipeline or stores its tile, the matrix cores of the unit idle, and every unit of
// the chip does so at the same time (the stores of all tiles of a round hit the memory system
// together).  Here a workgroup is half as large -- 256 lanes = 4 waves (2 x 2), macro tile 128
// (m) x 256 (n), wave tile 64 x 128 = 2 x 4 MFMA tiles = 128 accumulators per lane, at most 256
// registers per wave, 80 KiB of LDS -- so that TWO of them are resident on a compute unit, two
// waves per SIMD, each with its own barriers.  While one stores its tile or fetches the first
// stages of its next one, the other keeps the matrix cores busy, and one wave's DMA and LDS
// instructions issue under the other's matrix instructions.  The two workgroups that start
// together on a unit are put half a tile out of phase once, at the start of the launch: the
// one in the unit's second wave slot sleeps for half a main loop (the other has the matrix
// cores to itself meanwhile, so nothing is lost).
//
// Same operand layouts, fragment reads, DMA geometry and epilogue as mfma_tile_kernel; k is
// consumed in the same 64-byte stages.  LDS: B stages in a ring of 3 slots of 16 KiB (a slot is
// refilled right after the barrier that follows its last fragment reads, two stages ahead of
// its next use), A as pairs of stages [128 m][128 B] in 2 slots of 16 KiB.
//
// Pipeline, stage s (B in slot s % 3, A in pair slot (s / 2) % 2):
//   k-step 0: 8 MFMAs on the fragments of (s,0); under them the 10 LDS reads of (s,1)
//   wait until this wave's DMA of stage s+1 has landed and its LDS reads are complete; barrier
//   k-step 1: 8 MFMAs on (s,1); under them the 10 LDS reads of (s+1,0) and the DMA: 4
//             instructions of B of stage s+3 into slot s % 3 and, when s is odd, the 4 of the A
//             pair of stages s+3, s+4 into the pair slot stage s just stopped reading.
#pragma once

#include "mfma_tile.h"

namespace cig {
namespace tile {

constexpr int T2_TILE_M = 128;
constexpr int T2_LDS_BYTES = 3 * OPERAND_BYTES + 2 * (T2_TILE_M * 128);   // 80 KiB

template <typename Math, int BMODE, typename Epi>
__global__ __launch_bounds__(256, 2) void mfma_tile2_kernel(int M, int N, int tiles_m, int tiles_n,
                                                            int KTS, int k_bytes,
                                                            const char* __restrict__ A,
                                                            int64_t lda,
                                                            const char* __restrict__ B,
                                                            int64_t ldb, Epi epi,
                                                            int first_round, int skew_sleeps) {
  static_assert(BMODE == B_KN16 || BMODE == B_KN8, "K x N operands of 16-bit or 8-bit elements");
  typedef typename Math::acc_t acc_t;
  typedef BTile<BMODE> BT;
  constexpr int MT = 2, NW = 4, TILE_M = T2_TILE_M, RING = 3;
  constexpr int DMA_A = TILE_M / 8 / NW;   // 4 per wave and stage pair
  constexpr int DMA_B = 16 / NW;           // 4 per wave and stage
  constexpr int APAIR_BYTES = TILE_M * 128;
  constexpr int B_RING = RING * OPERAND_BYTES;
  typedef RowPairDmaT<1> PairDma;
  extern __shared__ __attribute__((aligned(1024))) char lds[];
  const int t = threadIdx.x;
  const int l = t & 63;
  const int w = __builtin_amdgcn_readfirstlane(t >> 6);
  const int wm = w >> 1, wn = w & 1;
  auto stamp = [&](int point) {
    if constexpr (epi_profiled<Epi>::value) {
      if (threadIdx.x == 0) {
        uint64_t* p = epi.stamps + (int64_t)blockIdx.x * 8 + 2 * point;
        p[0] = point == 0 ? ((uint64_t)__builtin_amdgcn_s_getreg((3 << 11) | 20) << 32) |
                                __builtin_amdgcn_s_getreg((31 << 11) | 4)
                          : __builtin_amdgcn_s_memtime();
        p[1] = __builtin_amdgcn_s_memrealtime();
      }
    }
  };
  stamp(0);
  // The phase shift.  Of the two workgroups that start together on a compute unit, the waves
  // of the second sit in wave slot 1 of their SIMDs (bit 0 of the hardware id register's wave
  // field): they sleep, a bounded number of times, before they touch anything.  Later
  // workgroups start whenever a predecessor ends and keep the shift.  (Where the hardware
  // places waves otherwise, the shift is missing or common to both: slower, never wrong.)
  if (blockIdx.x < first_round) {
    const uint32_t hw_id = __builtin_amdgcn_s_getreg((31 << 11) | 4);
    if (hw_id & 1u)
      for (int i = 0; i < skew_sleeps; ++i) __builtin_amdgcn_s_sleep(64);
  }

  int tm, tn;
  tile_of_workgroup(tiles_m, tiles_n, tm, tn);
  tm = __builtin_amdgcn_readfirstlane(tm);
  tn = __builtin_amdgcn_readfirstlane(tn);
  const int64_t m0 = (int64_t)tm * TILE_M, n0 = (int64_t)tn * BN;
  float epi_row_word = 0.0f, epi_col_word = 0.0f;
  if constexpr (epi_has_uniform_mode<Epi>::value) {
    epi_row_word = *epi.row_word();
    epi_col_word = *epi.col_word();
  }

  // ---- DMA sources (see mfma_tile_kernel) -------------------------------------------------------
  const char* a_tile = A + m0 * lda;
  const char* b_tile = B + n0 * Math::ELEM_BYTES;
  const int64_t b_kstep = (int64_t)(KB / Math::ELEM_BYTES) * ldb;
  const int a_last = (int)((M - 1 - m0) < (TILE_M - 1) ? (M - 1 - m0) : (TILE_M - 1));
  const int n_left = (int)((N - n0) < BN ? (N - n0) : BN);
  const int b_last = (n_left * Math::ELEM_BYTES + 15) / 16 - 1;
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
    b_voff[i] = (uint32_t)BT::dma_src(q >> 2, q & 3, l, ldb, b_last);
  }
  const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)lds;
  auto dma16 = [&](const char* base, uint32_t voff, uint32_t lds_dst) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :
                 : "s"(lds_dst), "v"(voff), "s"(base)
                 : "m0");
  };
  auto dma16z = [&](const char* base, uint32_t voff, uint32_t lds_dst, bool zero) {
    const char* src = zero ? zero_src : base + voff;
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off"
                 :
                 : "s"(lds_dst), "v"(src)
                 : "m0");
  };
  auto pair_piece = [&](int q) { return (l & 7) ^ ((4 * (q & 1) + (l >> 4)) & 7); };
  // B instruction d of stage `st` into ring slot `slot`; past the last stage the last one is
  // fetched again into a slot nobody reads any more (uniform wait counts)
  auto dma_b = [&](int st, int slot, int d, auto steady_const) {
    constexpr bool STEADY = decltype(steady_const)::value;
    if (!STEADY) st = st < KTS ? st : KTS - 1;
    const int q = DMA_B * w + d;
    const uint32_t dst = lds_base + slot * OPERAND_BYTES + BT::dma_lds(q >> 2, q & 3);
    if (STEADY)
      dma16(b_tile + (int64_t)st * b_kstep, b_voff[d], dst);
    else
      dma16z(b_tile + (int64_t)st * b_kstep, b_voff[d], dst,
             st == KTS - 1 && BT::dma_k(q >> 2, q & 3, l) * Math::ELEM_BYTES >= tail_k);
  };
  // A instruction d of the pair that holds stage `st` into pair slot `pslot`
  auto dma_a = [&](int st, int pslot, int d, auto steady_const) {
    constexpr bool STEADY = decltype(steady_const)::value;
    if (!STEADY) st = st < KTS ? st : KTS - 1;
    const int q = DMA_A * w + d;
    const uint32_t dst = lds_base + B_RING + pslot * APAIR_BYTES + PairDma::dma_lds(q >> 1, q & 1);
    if (STEADY)
      dma16(a_tile + (int64_t)(st >> 1) * 128, a_voff[d], dst);
    else
      dma16z(a_tile + (int64_t)(st >> 1) * 128, a_voff[d], dst,
             (st >> 1) == last_pair && pair_piece(q) >= pair_valid);
  };
  typedef std::integral_constant<bool, true> steady_t;
  typedef std::integral_constant<bool, false> drain_t;

  const int a_frag_row = wm * 32 * MT + (l & 31);
  const int g = l >> 5;
  constexpr int NREAD = MT + BT::NREADS;   // LDS reads per k-step: 2 + 8
  constexpr int NMFMA = 4 * MT;            // MFMAs per k-step: 8
  constexpr int READS_PER_SLOT = (NREAD + NMFMA - 1) / NMFMA;
  struct Frags {
    u32x4 a[MT];
    typename BT::piece_t b[BT::NREADS];
  };
  auto read_piece = [&](Frags& f, int slot, int pslot, int par, int kk, int r) {
    if (r < MT)
      f.a[r] = *reinterpret_cast<const u32x4*>(
          lds + B_RING + pslot * APAIR_BYTES + pair_off(a_frag_row + 32 * r, 4 * par + 2 * kk + g));
    else
      f.b[r - MT] = read_b_piece<BMODE>(lds + slot * OPERAND_BYTES, wn, r - MT, kk, l);
  };

  acc_t acc[MT][4];
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0;
  auto mfma_piece = [&](const Frags& f, int m) {
    const int j = m / MT;
    const int i = (j & 1) ? MT - 1 - m % MT : m % MT;
    acc[i][j] = Math::mfma(BT::bfrag(f.b, j, 0), Math::afrag(f.a[i], 0), acc[i][j]);
  };
  Frags f0, f1;
  auto wait_vmcnt = [](auto n_const) {
    constexpr int n = decltype(n_const)::value;
    __builtin_amdgcn_s_waitcnt(0x0f70 | (n & 15) | ((n >> 4) << 14));
  };

  // prologue, in the order the main loop keeps: B[0], A pair 0; B[1]; B[2], A pair 1
#pragma unroll
  for (int d = 0; d < DMA_B; ++d) dma_b(0, 0, d, drain_t{});
#pragma unroll
  for (int d = 0; d < DMA_A; ++d) dma_a(0, 0, d, drain_t{});
#pragma unroll
  for (int d = 0; d < DMA_B; ++d) dma_b(1, 1, d, drain_t{});
#pragma unroll
  for (int d = 0; d < DMA_B; ++d) dma_b(2, 2, d, drain_t{});
#pragma unroll
  for (int d = 0; d < DMA_A; ++d) dma_a(2, 1, d, drain_t{});
  wait_vmcnt(std::integral_constant<int, 2 * DMA_B + DMA_A>{});
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int r = 0; r < NREAD; ++r) read_piece(f0, 0, 0, 0, 0, r);
  stamp(1);

  int slot = 0, next_slot = 1;
  int pslot = 0, next_pslot = 1;
  auto stage = [&](int s, auto par_const, auto steady_const) {
    constexpr int PAR = decltype(par_const)::value;
    constexpr int NDMA = PAR ? DMA_B + DMA_A : DMA_B;
#pragma unroll
    for (int sl = 0; sl < NMFMA; ++sl) {
      mfma_piece(f0, sl);
#pragma unroll
      for (int r = sl * READS_PER_SLOT; r < (sl + 1) * READS_PER_SLOT; ++r)
        if (r < NREAD) read_piece(f1, slot, pslot, PAR, 1, r);
      __builtin_amdgcn_sched_barrier(0);
    }
    // Stage s+1 landed for this wave.  Still in flight, issued after what stage s+1 needs:
    // even s: B[s+2] and the A pair of stages s+2, s+3; odd s: B[s+2].  This wave's reads of
    // slot s % 3 (and, in an odd stage, of the A pair slot) are complete before any wave
    // refills them after the barrier.
    wait_vmcnt(std::integral_constant<int, PAR ? DMA_B : DMA_B + DMA_A>{});
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int sl = 0; sl < NMFMA; ++sl) {
      mfma_piece(f1, sl);
#pragma unroll
      for (int r = sl * READS_PER_SLOT; r < (sl + 1) * READS_PER_SLOT; ++r)
        if (r < NREAD) read_piece(f0, next_slot, PAR ? next_pslot : pslot, PAR ^ 1, 0, r);
      // one DMA instruction per slot in odd stages, one every second slot in even stages
      if (PAR ? true : (sl % 2 == 0)) {
        const int d = PAR ? sl : sl / 2;
        if (d < NDMA) {
          if (d < DMA_B)
            dma_b(s + 3, slot, d, steady_const);
          else
            dma_a(s + 3, pslot, d - DMA_B, steady_const);
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    slot = next_slot;
    next_slot = next_slot + 1 == RING ? 0 : next_slot + 1;
    if (PAR) {
      const int tmp = pslot;
      pslot = next_pslot;
      next_pslot = tmp;
    }
  };
  // Steady part: every stage the DMA reaches (up to s + 5) exists and its pair is whole.
  const int steady_end = (pair_valid < 8 && !(KTS & 1)) ? KTS - 2 : KTS;
  int s = 0;
  for (; s + 5 < steady_end; s += 2) {
    stage(s, std::integral_constant<int, 0>{}, steady_t{});
    stage(s + 1, std::integral_constant<int, 1>{}, steady_t{});
  }
  for (; s + 1 < KTS; s += 2) {
    stage(s, std::integral_constant<int, 0>{}, drain_t{});
    stage(s + 1, std::integral_constant<int, 1>{}, drain_t{});
  }
  if (KTS & 1) stage(KTS - 1, std::integral_constant<int, 0>{}, drain_t{});
  wait_vmcnt(std::integral_constant<int, 0>{});  // no DMA outlives the main loop
  __syncthreads();  // ... for any wave, and every wave is done reading the ring
  stamp(2);

  store_tile<Math, MT, NW, TILE_M>(epi, acc, lds, w, wm, wn, m0, n0, M, N, epi_row_word,
                                   epi_col_word);
  if constexpr (epi_profiled<Epi>::value) {
    wait_vmcnt(std::integral_constant<int, 0>{});
    stamp(3);
  }
}

// Launches the two-per-unit form.  No split-K (the caller keeps the other form for that).
template <typename Math, int BMODE, typename Epi>
void launch_tile2(cigemmContext* ctx, int64_t M, int64_t N, int64_t K_bytes, const void* A,
                  int64_t lda_bytes, const void* B, int64_t ldb_bytes, const Epi& epi) {
  auto kern = mfma_tile2_kernel<Math, BMODE, Epi>;
  static std::atomic<uint64_t> lds_set{0};
  if (!ensure_dynamic_lds(ctx, (const void*)kern, T2_LDS_BYTES, lds_set)) return;
  const int tiles_m = (int)((M + T2_TILE_M - 1) / T2_TILE_M), tiles_n = (int)((N + BN - 1) / BN);
  const int64_t kts = (K_bytes + KB - 1) / KB;
  const int cus = ctx->num_cus > 0 ? ctx->num_cus : 256;
  // half of one workgroup's main loop when it has the matrix cores to itself: 8 MFMAs of 32
  // cycles per k-step and wave plus a fifth for everything else, in sleeps of 4096 cycles
  int64_t sleeps = kts * 2 * 8 * 32 * 6 / 5 / 2 / 4096;
  if (sleeps > 64) sleeps = 64;
  ctx->last_tile_rows = T2_TILE_M;
  ctx->last_k_splits = 1;
  ctx->last_waves = 4;
  ctx->last_per_cu = 2;
  hipLaunchKernelGGL(kern, dim3((unsigned)(tiles_m * tiles_n)), dim3(256), T2_LDS_BYTES,
                     ctx->stream, (int)M, (int)N, tiles_m, tiles_n, (int)kts, (int)K_bytes,
                     static_cast<const char*>(A), lda_bytes, static_cast<const char*>(B),
                     ldb_bytes, epi, 2 * cus, (int)sleeps);
}

}  // namespace tile
}  // namespace cig
