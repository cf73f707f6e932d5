// Any-shape GEMM on the matrix cores, for the calls that the LDS-DMA tile kernel and the small
// fp32 kernel cannot take (an odd N, rows or pointers that are not 16-byte aligned, a K whose bytes
// are not a multiple of 16): the scalar any-shape kernel runs those at 30 (16-bit) to 45 (fp32)
// TFLOP/s, far below the tile kernel, and the library this path replaces has no such cliff
// (quantization/GEMM_bf16.cu:51-56 passes whatever m, n, k, lda, ldb it is given).
//
// One 128 x 128 output tile per 256-thread workgroup, four waves of 64 x 64 (2 x 2 MFMA tiles
// of 32 x 32), 64 bytes of k per step.  Operands are fetched in 16-byte pieces of a row, each
// with one unconditional vector load at whatever alignment the row has (the compiler is told
// the element's alignment only and emits what the target's unaligned-access mode allows) from
// an address clamped into the matrix; what a piece holds beyond the end of its row, of K or of
// the matrix is dropped in registers afterwards (no branch around a load: a wait at every join
// would keep the loads from overlapping the multiplies).  The pieces are held in registers
// while the previous step multiplies, and written to LDS as the rows
// they are: A, and B when it is N x K, as [row][64 B of k] with rows 80 bytes apart; a K x N
// operand as [k][128 columns] with rows 320 (16-bit), 160 (int8) or 544 (fp32) bytes apart.  MFMA operands
// of the first kind are read with one 16-byte read per lane (row l % 32, k offset 16 (l / 32) of
// a 32-byte chunk); a K x N operand goes through the transposing reads ds_read_b64_tr_b16 /
// _tr_b8 (within 16 lanes, lane i supplies the address of 8 bytes of k row i / 4 -- i / 2 for
// bytes -- and receives the k-values of column i; fp32: four single-float reads, one per k row).
// The row pitches spread the rows that one
// read instruction touches over all banks.  Outputs leave through the element-wise epilogues of
// the scalar any-shape kernel, so every output type and scale mode is served and nothing is
// assumed about the alignment of C either.
//
// Arithmetic: 16-bit and int8 products exact, fp32 (int32) accumulation inside the MFMA in its
// own order -- int8 results equal the CPU loop bit for bit, 16-bit results are within the same
// K-scaled bound as the tile kernel's; fp32 (v_mfma_f32_32x32x2_f32: true fp32 products and sums)
// within the same scaled 1e-5 tolerance of the CPU loop as the fp32 tile kernel's.  Only the
// scalar kernel (CIGEMM_ALGO_GENERIC) reproduces the CPU loop's fp32 bits.
#include "common.h"
#include "mfma_tile.h"

namespace cig {
namespace {

constexpr int RT = 128;        // tile edge
constexpr int RK = 64;         // bytes of k per step
constexpr int RROW = RK + 16;  // LDS row pitch of a k-contiguous operand

template <int ELEM_BYTES>
struct RaggedElem;
template <>
struct RaggedElem<2> {
  typedef uint16_t type;
  static constexpr int KN_PITCH = 320;  // [32 k][256 B], rows 16 banks apart
};
template <>
struct RaggedElem<1> {
  typedef uint8_t type;
  static constexpr int KN_PITCH = 160;  // [64 k][128 B], 8 consecutive rows 8 banks apart
};
template <>
struct RaggedElem<4> {
  typedef uint32_t type;                // fp32, moved as bits
  static constexpr int KN_PITCH = 544;  // [16 k][512 B], rows k and k + 4 half the banks apart
};

// One 16-byte piece = elements [col, col + CE) of row `row` of a row-major matrix with `rows`
// rows of `cols` elements, zero outside the matrix, in two steps so that the load is one
// unconditional instruction that can stay in flight while the previous step multiplies:
// load_piece reads 16 bytes that lie inside the matrix whatever the piece (row clamped to the
// last one; a piece that crosses the end of its row is replaced by the row's last 16 bytes),
// trim_piece, applied when the value is needed, moves those down so that element `col` comes
// first and zeroes what lies outside.  Needs cols >= CE.
template <typename T>
__device__ __forceinline__ u32x4 load_piece(const T* __restrict__ P, int64_t ld, int64_t row,
                                            int64_t rows, int64_t col, int64_t cols) {
  constexpr int CE = 16 / (int)sizeof(T);
  const int64_t r = row < rows ? row : rows - 1;
  const int64_t c = col + CE <= cols ? col : cols - CE;
  u32x4 v;
  __builtin_memcpy(&v, P + r * ld + c, 16);
  return v;
}
template <typename T>
__device__ __forceinline__ u32x4 trim_piece(u32x4 v, int64_t row, int64_t rows, int64_t col,
                                            int64_t cols) {
  constexpr int CE = 16 / (int)sizeof(T);
  const bool inside = row < rows && col < cols;
  const int s = col + CE > cols && inside ? (int)(col - (cols - CE)) * 8 * (int)sizeof(T) : 0;
  const int s1 = s & 63;  // bits to move down: 0 <= s < 128
  const uint64_t lo = v[0] | ((uint64_t)v[1] << 32), hi = v[2] | ((uint64_t)v[3] << 32);
  const uint64_t lo1 = (lo >> s1) | ((hi << 1) << (63 - s1)), hi1 = hi >> s1;
  const uint64_t lo2 = s >= 64 ? hi1 : lo1, hi2 = s >= 64 ? 0 : hi1;
  const u32x4 r = {inside ? (uint32_t)lo2 : 0u, inside ? (uint32_t)(lo2 >> 32) : 0u,
                   inside ? (uint32_t)hi2 : 0u, inside ? (uint32_t)(hi2 >> 32) : 0u};
  return r;
}
// The same piece element by element, for a matrix narrower than a piece.
template <typename T>
__device__ __forceinline__ u32x4 fetch_piece_narrow(const T* __restrict__ P, int64_t ld,
                                                    int64_t row, int64_t rows, int64_t col,
                                                    int64_t cols) {
  constexpr int CE = 16 / (int)sizeof(T);
  T tmp[CE];
#pragma unroll
  for (int e = 0; e < CE; ++e)
    tmp[e] = row < rows && col + e < cols ? P[row * ld + col + e] : (T)0;
  u32x4 v;
  __builtin_memcpy(&v, tmp, 16);
  return v;
}

// Split-K: the accumulators of one K range, stored raw (fp32 or int32 bits) to
// base[split * split_stride + r * ld + c]; a second kernel sums the ranges in order and applies
// the real epilogue, one element per lane.
struct EpiPartialElem {
  uint32_t* base;
  int64_t ld;
  int64_t split_stride;
  template <typename T>
  __device__ __forceinline__ void operator()(int64_t r, int64_t c, T acc) const {
    base[r * ld + c] = __builtin_bit_cast(uint32_t, acc);
  }
};
template <typename Epi>
__device__ __forceinline__ Epi any_epilogue_of_split(const Epi& e, int) { return e; }
__device__ __forceinline__ EpiPartialElem any_epilogue_of_split(const EpiPartialElem& e, int split) {
  return EpiPartialElem{e.base + split * e.split_stride, e.ld, e.split_stride};
}

template <typename Scalar, typename Epi>
__global__ __launch_bounds__(256) void any_reduce_kernel(int64_t M, int64_t N, int splits,
                                                         const uint32_t* __restrict__ part,
                                                         int64_t split_stride, Epi epi) {
  const int64_t total = M * N;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total;
       i += (int64_t)gridDim.x * 256) {
    // all ranges are read before the first add waits for one (splits <= 16)
    uint32_t v[16];
#pragma unroll
    for (int sp = 0; sp < 16; ++sp)
      if (sp < splits) v[sp] = part[sp * split_stride + i];
    Scalar sum = __builtin_bit_cast(Scalar, v[0]);
#pragma unroll
    for (int sp = 1; sp < 16; ++sp)
      if (sp < splits) sum += __builtin_bit_cast(Scalar, v[sp]);
    epi(i / N, i % N, sum);
  }
}

template <typename Math, bool B_NK, typename Epi>
__global__ __launch_bounds__(256) void mfma_any_kernel(int64_t M, int64_t N, int64_t K,
                                                       const void* __restrict__ Av, int64_t lda,
                                                       const void* __restrict__ Bv, int64_t ldb,
                                                       Epi epi_all, int tiles_m, int tiles_n,
                                                       int64_t k_range) {
  // blockIdx.y = K range (split launches only): k in [y * k_range, min(K, (y + 1) * k_range)),
  // k_range a multiple of the step; the rest of the kernel sees that range as its K
  const Epi epi = any_epilogue_of_split(epi_all, (int)blockIdx.y);
  const int64_t k_begin = (int64_t)blockIdx.y * k_range;
  K = K < k_begin + k_range ? K : k_begin + k_range;
  typedef RaggedElem<Math::ELEM_BYTES> E;
  typedef typename E::type elem_t;
  typedef typename Math::acc_t acc_t;
  constexpr int EB = Math::ELEM_BYTES;
  constexpr int KE = RK / EB;               // elements of k per step: 32, 64 or (fp32) 16
  constexpr int CE = 16 / EB;               // elements per 16-byte piece
  constexpr int KN_PIECES = RT * EB / 16;   // pieces per k row of a K x N tile: 16, 8 or 32
  constexpr int BP = E::KN_PITCH;
  static_assert(RT * RROW >= KE * BP, "both B layouts fit the same LDS array");
  __shared__ __attribute__((aligned(16))) unsigned char As[RT * RROW];
  __shared__ __attribute__((aligned(16))) unsigned char Bs[RT * RROW];
  const elem_t* __restrict__ A = static_cast<const elem_t*>(Av);
  const elem_t* __restrict__ B = static_cast<const elem_t*>(Bv);

  const int t = threadIdx.x, l = t & 63, w = t >> 6;
  const int wm = w >> 1, wn = w & 1;
  // Workgroups go to the 8 XCDs round-robin; each XCD gets a contiguous range of logical ids,
  // which walk the tile grid in column-major groups of 8 tile rows: the tiles resident on one
  // XCD at a time (about three per compute unit) share A and B panels in that XCD's L2.
  int tm, tn;
  {
    constexpr int64_t XCDS = 8, GROUP_M = 8;
    const int64_t nwg = (int64_t)tiles_m * tiles_n, pid = blockIdx.x;
    const int64_t xcd = pid % XCDS, local = pid / XCDS, base = nwg / XCDS, rem = nwg % XCDS;
    const int64_t wg = xcd * base + (xcd < rem ? xcd : rem) + local;
    const int64_t per_group = GROUP_M * tiles_n, first_m = wg / per_group * GROUP_M;
    const int64_t gsize = tiles_m - first_m < GROUP_M ? tiles_m - first_m : GROUP_M;
    tm = (int)(first_m + wg % per_group % gsize);
    tn = (int)(wg % per_group / gsize);
  }
  const int64_t m0 = (int64_t)tm * RT, n0 = (int64_t)tn * RT;

  // 512 pieces per operand and step, two per thread: piece c = t + 256 i.
  // k-contiguous operand: row c / 4, piece c % 4 of its 64 bytes; K x N: k row c / KN_PIECES,
  // piece c % KN_PIECES of its 128 columns.
  // NARROW: K, or the N of a K x N operand, is shorter than a piece (uniform over the launch)
  u32x4 ra[2], rb[2];
  auto fetch = [&](int64_t k0, auto narrow) {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int c = t + 256 * i;
      if constexpr (decltype(narrow)::value) {
        ra[i] = fetch_piece_narrow(A, lda, m0 + (c >> 2), M, k0 + (c & 3) * CE, K);
        if (B_NK)
          rb[i] = fetch_piece_narrow(B, ldb, n0 + (c >> 2), N, k0 + (c & 3) * CE, K);
        else
          rb[i] = fetch_piece_narrow(B, ldb, k0 + c / KN_PIECES, K, n0 + (c % KN_PIECES) * CE, N);
      } else {
        ra[i] = load_piece(A, lda, m0 + (c >> 2), M, k0 + (c & 3) * CE, K);
        if (B_NK)
          rb[i] = load_piece(B, ldb, n0 + (c >> 2), N, k0 + (c & 3) * CE, K);
        else
          rb[i] = load_piece(B, ldb, k0 + c / KN_PIECES, K, n0 + (c % KN_PIECES) * CE, N);
      }
    }
  };
  // writes the pieces fetched for the step at k0 to LDS
  auto stash = [&](int64_t k0, auto narrow) {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int c = t + 256 * i;
      u32x4 va = ra[i], vb = rb[i];
      if constexpr (!decltype(narrow)::value) {
        va = trim_piece<elem_t>(va, m0 + (c >> 2), M, k0 + (c & 3) * CE, K);
        if (B_NK)
          vb = trim_piece<elem_t>(vb, n0 + (c >> 2), N, k0 + (c & 3) * CE, K);
        else
          vb = trim_piece<elem_t>(vb, k0 + c / KN_PIECES, K, n0 + (c % KN_PIECES) * CE, N);
      }
      *reinterpret_cast<u32x4*>(As + (c >> 2) * RROW + (c & 3) * 16) = va;
      if (B_NK)
        *reinterpret_cast<u32x4*>(Bs + (c >> 2) * RROW + (c & 3) * 16) = vb;
      else
        *reinterpret_cast<u32x4*>(Bs + (c / KN_PIECES) * BP + (c % KN_PIECES) * 16) = vb;
    }
  };

  acc_t acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0;

  const unsigned char* a_frag = As + (64 * wm + (l & 31)) * RROW + 16 * (l >> 5);
  const unsigned char* b_frag = Bs + (64 * wn + (l & 31)) * RROW + 16 * (l >> 5);
  // K x N: byte address, within Bs, of the 8 bytes this lane supplies to the first transposing
  // read of column tile 0, k block 0
  const unsigned char* b_tr =
      EB == 2 ? Bs + (8 * (l >> 5) + ((l & 15) >> 2)) * BP +
                    (64 * wn + 16 * ((l >> 4) & 1) + 4 * (l & 3)) * 2
              : Bs + (16 * (l >> 5) + ((l & 15) >> 1)) * BP + 64 * wn + 16 * ((l >> 4) & 1) +
                    8 * (l & 1);
  auto b_fragment = [&](int j, int kk) -> u32x4 {
    if constexpr (B_NK) {
      return *reinterpret_cast<const u32x4*>(b_frag + 32 * j * RROW + 32 * kk);
    } else if constexpr (EB == 4) {
      // four single floats: column n of k rows 8 kk + 4 (l / 32) + e
      const unsigned char* p = Bs + (8 * kk + 4 * (l >> 5)) * BP + (64 * wn + 32 * j + (l & 31)) * 4;
      const u32x4 v = {*reinterpret_cast<const uint32_t*>(p),
                       *reinterpret_cast<const uint32_t*>(p + BP),
                       *reinterpret_cast<const uint32_t*>(p + 2 * BP),
                       *reinterpret_cast<const uint32_t*>(p + 3 * BP)};
      return v;
    } else if constexpr (EB == 2) {
      // an MFMA's 16 k rows start at row 16 kk; the second read takes the rows 4 further on
      const unsigned char* p = b_tr + 16 * kk * BP + 64 * j;
      const i16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((tile::lds_i16x4*)p);
      const i16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((tile::lds_i16x4*)(p + 4 * BP));
      return __builtin_shufflevector(__builtin_bit_cast(u32x2, lo), __builtin_bit_cast(u32x2, hi),
                                     0, 1, 2, 3);
    } else {
      // 32 k rows per MFMA; the second read takes the rows 8 further on
      const unsigned char* p = b_tr + 32 * kk * BP + 32 * j;
      const i32x2 lo = __builtin_amdgcn_ds_read_tr8_b64_v2i32((tile::lds_i32x2*)p);
      const i32x2 hi = __builtin_amdgcn_ds_read_tr8_b64_v2i32((tile::lds_i32x2*)(p + 8 * BP));
      return __builtin_shufflevector(__builtin_bit_cast(u32x2, lo), __builtin_bit_cast(u32x2, hi),
                                     0, 1, 2, 3);
    }
  };

  auto run = [&](auto narrow) {
    fetch(k_begin, narrow);
    for (int64_t k0 = k_begin; k0 < K; k0 += KE) {
      stash(k0, narrow);
      __syncthreads();
      if (k0 + KE < K) fetch(k0 + KE, narrow);  // in flight while this step multiplies
#pragma unroll
      for (int kk = 0; kk < 2; ++kk) {
        u32x4 af[2], bf[2];
#pragma unroll
        for (int i = 0; i < 2; ++i) {
          af[i] = *reinterpret_cast<const u32x4*>(a_frag + 32 * i * RROW + 32 * kk);
          bf[i] = b_fragment(i, kk);
        }
        if constexpr (EB == 4) {
          // 8 k per 32-byte chunk: the MFMA takes one float per lane and operand (lanes 0-31
          // k, lanes 32-63 k + 4), so element e of the two fragments feeds MFMA e
#pragma unroll
          for (int e = 0; e < 4; ++e)
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
              for (int j = 0; j < 2; ++j)
                acc[i][j] = Math::mfma(Math::afrag(af[i], e), Math::afrag(bf[j], e), acc[i][j]);
        } else {
#pragma unroll
          for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j) acc[i][j] = Math::mfma(af[i], bf[j], acc[i][j]);
        }
      }
      __syncthreads();
    }
  };
  if (K < CE || (!B_NK && N < CE))
    run(std::true_type{});
  else
    run(std::false_type{});

  // acc[i][j][4 q + e] = C[m0 + 64 wm + 32 i + 8 q + 4 (l / 32) + e][n0 + 64 wn + 32 j + l % 32]
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int64_t gn = n0 + 64 * wn + 32 * j + (l & 31);
      if (gn >= N) continue;
#pragma unroll
      for (int q = 0; q < 4; ++q)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int64_t gm = m0 + 64 * wm + 32 * i + 8 * q + 4 * (l >> 5) + e;
          if (gm < M) epi(gm, gn, acc[i][j][4 * q + e]);
        }
    }
}

// K ranges for a problem of few tiles (a decode or small-batch shape that no aligned kernel
// takes): about three workgroups per compute unit are resident, so enough ranges to fill those
// places, each of at least four steps, at most 16, partials within the workspace.  N = 8191,
// K = 8192, M = 1 (64 tiles): 255 us unsplit.
template <typename Math>
int any_splits(const cigemmContext* ctx, int64_t M, int64_t N, int64_t K, int64_t tiles) {
  constexpr int KE = RK / Math::ELEM_BYTES;
  const int cus = ctx->num_cus > 0 ? ctx->num_cus : 256;
  if (!ctx->workspace || tiles * 2 > 3 * (int64_t)cus) return 1;  // fewer than two ranges fit
  const int64_t steps = (K + KE - 1) / KE;
  int64_t s = 3 * (int64_t)cus / tiles;
  if (s > 16) s = 16;
  if (s > steps / 4) s = steps / 4;
  while (s > 1 && (size_t)s * (size_t)M * (size_t)N * 4 > ctx->ws_partial_bytes) --s;
  return s < 1 ? 1 : (int)s;
}

// Returns the number of K ranges the problem was run in.
template <typename Math, bool B_NK, typename Epi>
int launch_any(cigemmContext* ctx, int64_t M, int64_t N, int64_t K, const void* A, int64_t lda,
               const void* B, int64_t ldb, const Epi& epi) {
  typedef typename Math::scalar_t scalar_t;
  constexpr int KE = RK / Math::ELEM_BYTES;
  const int tiles_m = (int)((M + RT - 1) / RT), tiles_n = (int)((N + RT - 1) / RT);
  const int64_t tiles = (int64_t)tiles_m * tiles_n;
  int splits = any_splits<Math>(ctx, M, N, K, tiles);
  // steps per range, rounded up; ranges that would start past K are dropped
  const int64_t steps = (K + KE - 1) / KE;
  const int64_t k_range = splits > 1 ? (steps + splits - 1) / splits * KE : (K > 0 ? K : 1);
  if (splits > 1) splits = (int)((K + k_range - 1) / k_range);
  if (splits <= 1) {
    hipLaunchKernelGGL((mfma_any_kernel<Math, B_NK, Epi>), dim3((unsigned)tiles), dim3(256), 0,
                       ctx->stream, M, N, K, A, lda, B, ldb, epi, tiles_m, tiles_n, k_range);
    return 1;
  }
  uint32_t* ws = static_cast<uint32_t*>(ctx->workspace);
  hipLaunchKernelGGL((mfma_any_kernel<Math, B_NK, EpiPartialElem>),
                     dim3((unsigned)tiles, (unsigned)splits), dim3(256), 0, ctx->stream, M, N, K, A,
                     lda, B, ldb, EpiPartialElem{ws, N, M * N}, tiles_m, tiles_n, k_range);
  const int64_t blocks = (M * N + 255) / 256;
  const int cus = ctx->num_cus > 0 ? ctx->num_cus : 256;
  hipLaunchKernelGGL((any_reduce_kernel<scalar_t, Epi>),
                     dim3((unsigned)(blocks < 8 * (int64_t)cus ? blocks : 8 * (int64_t)cus)),
                     dim3(256), 0, ctx->stream, M, N, splits, ws, M * N, epi);
  return splits;
}

// "<name>" or "<name>_splitk", kept in the context
void set_any_name(cigemmContext* ctx, const char* name, int splits) {
  snprintf(ctx->kernel_name, sizeof(ctx->kernel_name), "%s%s", name, splits > 1 ? "_splitk" : "");
  ctx->last_kernel = ctx->kernel_name;
}

template <bool B_NK>
int launch_any_i8_layout(cigemmContext* ctx, int64_t M, int64_t N, int64_t K, const int8_t* A,
                         int64_t lda, const int8_t* B, int64_t ldb, int32_t* C, int64_t ldc,
                         const DequantArgs* dq) {
  if (!dq) return launch_any<tile::MathI8, B_NK>(ctx, M, N, K, A, lda, B, ldb, EpiStoreI32{C, ldc});
  const bool dump = dq->acc_out != nullptr;
#define CIG_DQ(OB, DA)                                                                        \
  launch_any<tile::MathI8, B_NK>(ctx, M, N, K, A, lda, B, ldb,                                 \
                                 EpiDequant<OB, DA>{dq->out, dq->ldo, dq->sa, dq->sb,          \
                                                    dq->sa_vec, dq->sb_vec, dq->acc_out,       \
                                                    dq->ldacc})
  if (dq->out_bf16) return dump ? CIG_DQ(true, true) : CIG_DQ(true, false);
  return dump ? CIG_DQ(false, true) : CIG_DQ(false, false);
#undef CIG_DQ
}

// one workgroup per tile, in a one-dimensional grid
bool any_shape_ok(int64_t M, int64_t N) {
  return M > 0 && N > 0 && ((M + RT - 1) / RT) * ((N + RT - 1) / RT) <= 2147483647LL &&
         (M + RT - 1) / RT <= 2147483647LL && (N + RT - 1) / RT <= 2147483647LL;
}

}  // namespace

bool launch_mfma_any_16(cigemmContext* ctx, bool bf16, int64_t M, int64_t N, int64_t K,
                        const uint16_t* A, int64_t lda, const uint16_t* B, int64_t ldb,
                        uint16_t* C, int64_t ldc) {
  if (!any_shape_ok(M, N)) return false;
  if (bf16)
    set_any_name(ctx, "bf16_mfma_any_128x128x32",
                 launch_any<tile::MathBF16, false>(ctx, M, N, K, A, lda, B, ldb,
                                                   EpiStore16<BF16>{C, ldc}));
  else
    set_any_name(ctx, "f16_mfma_any_128x128x32",
                 launch_any<tile::MathF16, false>(ctx, M, N, K, A, lda, B, ldb,
                                                  EpiStore16<F16>{C, ldc}));
  return true;
}

bool launch_mfma_any_f32(cigemmContext* ctx, int64_t M, int64_t N, int64_t K, const float* A,
                         int64_t lda, const float* B, int64_t ldb, float* C, int64_t ldc,
                         const BiasAct* ba) {
  if (!any_shape_ok(M, N)) return false;
  if (ba)
    set_any_name(ctx, "f32_mfma_any_128x128x16_bias_act",
                 launch_any<tile::MathF32, false>(ctx, M, N, K, A, lda, B, ldb,
                                                  EpiBiasActF32{C, ldc, ba->bias, ba->relu}));
  else
    set_any_name(ctx, "f32_mfma_any_128x128x16",
                 launch_any<tile::MathF32, false>(ctx, M, N, K, A, lda, B, ldb,
                                                  EpiStoreF32{C, ldc}));
  return true;
}

bool launch_mfma_any_i8(cigemmContext* ctx, int64_t M, int64_t N, int64_t K, const int8_t* A,
                        int64_t lda, const int8_t* B, int64_t ldb, bool b_nk, int32_t* C,
                        int64_t ldc, const DequantArgs* dq) {
  if (!any_shape_ok(M, N)) return false;
  const int splits = b_nk ? launch_any_i8_layout<true>(ctx, M, N, K, A, lda, B, ldb, C, ldc, dq)
                          : launch_any_i8_layout<false>(ctx, M, N, K, A, lda, B, ldb, C, ldc, dq);
  set_any_name(ctx,
               b_nk ? (dq ? "i8_mfma_any_128x128x64_nk_dequant" : "i8_mfma_any_128x128x64_nk")
                    : (dq ? "i8_mfma_any_128x128x64_kn_dequant" : "i8_mfma_any_128x128x64_kn"),
               splits);
  return true;
}

}  // namespace cig
