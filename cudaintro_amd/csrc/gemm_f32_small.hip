// fp32 GEMM for problems too small (or too narrow) to fill the chip with 256-column tiles:
// one 32x32 output tile per 256-lane workgroup, the k range split over the four waves
// (each wave: v_mfma_f32_32x32x2_f32 on operands loaded straight from global memory, no
// workgroup-wide staging), the four partial tiles summed through LDS in wave order
// (deterministic), then bias / activation and the store.
//
// A vector-memory instruction costs the issuing wave some 30 cycles of matrix-core issue, so
// their number per MFMA is what bounds the loop.  A fragments are one 16-byte load per lane
// and 8-deep k block.  B fragments (lane (n, g) needs B[k][n] for four k) are four 4-byte
// loads per block -- or, when B's rows allow 16-byte loads (BVEC), one: the wave fetches the
// block's 8 x 32 sub-tile as 64 x 16 bytes, passes it through a private 1 KiB of LDS (LDS
// instructions are almost free next to MFMAs) and reads its four values back.
//
// 512^3 gives 256 workgroups instead of the 16 of the 64x256 tile.  Outputs of at most 16
// columns have a form of their own below.
//
// Ragged M and N: loads past the edge re-read the last valid row / column, stores are
// masked.  K must be a multiple of 8 and A's rows 16-byte aligned.
#include "common.h"

namespace cig {
namespace {

constexpr int ST = 32;        // tile edge = one MFMA tile
constexpr int RED_LD = 36;    // floats per row of a partial tile in LDS (16-byte rows, padded)

constexpr int BSTG_LD = 40;   // floats per k row of the B staging block: rows 4 apart (the two
                              // halves of a wave) fall 32 banks apart

template <bool HAS_BIAS, bool RELU, bool BVEC>
__global__ __launch_bounds__(256) void f32_small_kernel(int M, int N, int K, int tiles_n,
                                                        const float* __restrict__ A, int64_t lda,
                                                        const float* __restrict__ B, int64_t ldb,
                                                        float* __restrict__ C, int64_t ldc,
                                                        const float* __restrict__ bias) {
  __shared__ __attribute__((aligned(16))) float red[4][ST][RED_LD];
  __shared__ __attribute__((aligned(16))) float bstg[BVEC ? 4 : 1][BVEC ? 2 : 1][8][BSTG_LD];
  const int t = threadIdx.x;
  const int w = t >> 6, l = t & 63;
  const int r = l & 31, h = l >> 5;
  const int tm = blockIdx.x / tiles_n, tn = blockIdx.x % tiles_n;
  const int m0 = tm * ST, n0 = tn * ST;

  // Lane (r, h) feeds row m0+r of A and column n0+r of B at k = kb + 4h + e, e = 0..3,
  // for every 8-deep block kb of its wave's share of K.
  const int row = min(m0 + r, M - 1);
  const int col = min(n0 + r, N - 1);
  const int nblk = K >> 3;
  const int b0 = (int)((int64_t)w * nblk / 4), b1 = (int)((int64_t)(w + 1) * nblk / 4);
  const float* ap = A + (int64_t)row * lda + 4 * h + 8 * (int64_t)b0;
  const float* bp = B + (4 * h + 8 * (int64_t)b0) * ldb + col;

  f32x16 acc;
#pragma unroll
  for (int i = 0; i < 16; ++i) acc[i] = 0.0f;

  // BVEC: lane l fetches B[8 b + l / 8][n0 + 4 (l % 8) .. + 3]; N is a multiple of 4 there, so a
  // quad is inside or outside as a whole (outside: the last valid quad again, never stored)
  const int vq = min(n0 + 4 * (l & 7), N - 4);
  const float* bvp = B + (8 * (int64_t)b0 + (l >> 3)) * ldb + vq;
  // one 8-deep k block: fragments in, four MFMAs
  auto block = [&](int b) {
    const f32x4 a = *reinterpret_cast<const f32x4*>(ap);
    float x0, x1, x2, x3;
    if constexpr (BVEC) {
      float(*st)[BSTG_LD] = bstg[w][b & 1];
      *reinterpret_cast<f32x4*>(&st[l >> 3][4 * (l & 7)]) = *reinterpret_cast<const f32x4*>(bvp);
      // the same wave reads what it wrote: LDS serves a wave's instructions in order
      x0 = st[4 * h][r], x1 = st[4 * h + 1][r], x2 = st[4 * h + 2][r], x3 = st[4 * h + 3][r];
      bvp += 8 * ldb;
    } else {
      x0 = bp[0], x1 = bp[ldb], x2 = bp[2 * ldb], x3 = bp[3 * ldb];
      bp += 8 * ldb;
    }
    // (B fragment, A fragment): the lane then holds four consecutive columns of one row.
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(x0, a[0], acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(x1, a[1], acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(x2, a[2], acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(x3, a[3], acc, 0, 0, 0);
    ap += 8;
  };
  int b = b0;
  if (BVEC) {
    // four blocks at a time, so that their loads are in flight together (with the strided
    // B loads the plain loop measures 3 % faster)
    for (; b + 4 <= b1; b += 4) {
#pragma unroll
      for (int u = 0; u < 4; ++u) block(b + u);
    }
  }
  for (; b < b1; ++b) block(b);

  // acc[4q+e] is C[m0 + r][n0 + 8q + 4h + e].
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const f32x4 v = {acc[4 * q], acc[4 * q + 1], acc[4 * q + 2], acc[4 * q + 3]};
    *reinterpret_cast<f32x4*>(&red[w][r][8 * q + 4 * h]) = v;
  }
  __syncthreads();

  const int om = t >> 3, on = (t & 7) * 4;
  f32x4 s = *reinterpret_cast<const f32x4*>(&red[0][om][on]);
#pragma unroll
  for (int ww = 1; ww < 4; ++ww) {
    const f32x4 p = *reinterpret_cast<const f32x4*>(&red[ww][om][on]);
#pragma unroll
    for (int e = 0; e < 4; ++e) s[e] = __fadd_rn(s[e], p[e]);
  }
  const int gm = m0 + om, gn = n0 + on;
  if (gm >= M) return;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    if (HAS_BIAS) s[e] = __fadd_rn(s[e], bias[min(gn + e, N - 1)]);
    if (RELU) s[e] = fmaxf(0.0f, s[e]);
  }
  float* out = C + (int64_t)gm * ldc + gn;
  if (gn + 3 < N && ((reinterpret_cast<uintptr_t>(out) & 15) == 0)) {
    *reinterpret_cast<f32x4*>(out) = s;
  } else {
#pragma unroll
    for (int e = 0; e < 4; ++e)
      if (gn + e < N) out[e] = s[e];
  }
}

// N <= 16 (the 10-wide output layer, MNIST/mnist_nn.cu:36-49): the 32x32 tile above spends
// two thirds of its MFMA time on padding columns and four of its five loads per block on B.
// Here a workgroup covers 16 * RB rows with v_mfma_f32_16x16x4_f32; the k range is split over
// the four waves as above and every wave keeps its share of B (at most 16 * NB k, 4 NB
// registers) in registers, so the loop issues one 16-byte load of A per four MFMAs.  K a
// multiple of 16.  20000 x 512 x 10 + bias: 14.4 us with the 32x32 form, 13.0 with this one
// and strided loads of B, 11.8 with B staged through LDS (3.5 TB/s of activations).
constexpr int NT = 16;        // narrow tile: rows per MFMA tile and padded columns
constexpr int NRED_LD = 20;   // floats per row of a partial tile in LDS (16-byte rows, padded)

template <int NB, int RB, bool STAGE_B>
__global__ __launch_bounds__(256) void f32_narrow_kernel(int M, int N, int K,
                                                         const float* __restrict__ A, int64_t lda,
                                                         const float* __restrict__ B, int64_t ldb,
                                                         float* __restrict__ C, int64_t ldc,
                                                         const float* __restrict__ bias, int relu) {
  __shared__ __attribute__((aligned(16))) float red[4][RB][NT][NRED_LD];
  const int t = threadIdx.x;
  const int w = __builtin_amdgcn_readfirstlane(t >> 6), l = t & 63;
  const int c = l & 15, g = l >> 4;
  const int m0 = blockIdx.x * (NT * RB);
  const int nblk = K >> 4;
  const int b0 = (int)((int64_t)w * nblk / 4), b1 = (int)((int64_t)(w + 1) * nblk / 4);
  const int nb = b1 - b0;  // <= NB (the launcher checks)

  // Lane (c, g) feeds column c of B and row c of each 16-row block of A at
  // k = 16 b + 4 g + e, e = 0..3, for every 16-deep block b of its wave's share of K.
  float wv[NB][4];
  if constexpr (STAGE_B) {
    // B is contiguous (ldb == N) and 16-byte aligned: the wave's share, rows 16 b0 .. 16 b1 - 1,
    // is one aligned run of 16 nb N floats.  It comes in as 16-byte loads (a fifth of the
    // instructions of the strided 4-byte loads below for N = 10), passes through the wave's
    // own piece of LDS and is read back by (k, column).  The same wave reads what it wrote:
    // LDS serves a wave's instructions in order.
    extern __shared__ __attribute__((aligned(16))) float bstage[];
    float* st = bstage + w * (NB * 16 * N);
    const f32x4* src = reinterpret_cast<const f32x4*>(B + 16 * (int64_t)b0 * N);
    const int nquads = nb * 4 * N;
    for (int q = l; q < nquads; q += 64) *reinterpret_cast<f32x4*>(st + 4 * q) = src[q];
#pragma unroll
    for (int b = 0; b < NB; ++b)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        wv[b][e] = 0.0f;
        if (b < nb) {
          const float v = st[(16 * b + 4 * g + e) * N + min(c, N - 1)];
          wv[b][e] = c < N ? v : 0.0f;
        }
      }
  } else {
    const float* bp = B + (16 * (int64_t)b0 + 4 * g) * ldb + min(c, N - 1);
#pragma unroll
    for (int b = 0; b < NB; ++b)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        wv[b][e] = 0.0f;
        if (b < nb) {
          const float v = bp[(16 * (int64_t)b + e) * ldb];
          wv[b][e] = c < N ? v : 0.0f;  // padding columns multiply by zero and are never stored
        }
      }
  }
  const float* ap[RB];
  f32x4 acc[RB];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    const int row = min(m0 + NT * rb + c, M - 1);
    ap[rb] = A + (int64_t)row * lda + 16 * (int64_t)b0 + 4 * g;
    acc[rb] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
  }
#pragma unroll
  for (int b = 0; b < NB; ++b) {
    if (b < nb) {
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) {
        const f32x4 a = *reinterpret_cast<const f32x4*>(ap[rb] + 16 * b);
        // (B fragment, A fragment): the lane then holds four consecutive columns of one row
#pragma unroll
        for (int e = 0; e < 4; ++e)
          acc[rb] = __builtin_amdgcn_mfma_f32_16x16x4f32(wv[b][e], a[e], acc[rb], 0, 0, 0);
      }
    }
  }
  // acc[rb][e] is C[m0 + 16 rb + c][4 g + e].
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) *reinterpret_cast<f32x4*>(&red[w][rb][c][4 * g]) = acc[rb];
  __syncthreads();

  if (t >= RB * 64) return;
  const int orb = t >> 6, om = (t >> 2) & 15, on = (t & 3) * 4;
  f32x4 s = *reinterpret_cast<const f32x4*>(&red[0][orb][om][on]);
#pragma unroll
  for (int ww = 1; ww < 4; ++ww) {
    const f32x4 p = *reinterpret_cast<const f32x4*>(&red[ww][orb][om][on]);
#pragma unroll
    for (int e = 0; e < 4; ++e) s[e] = __fadd_rn(s[e], p[e]);
  }
  const int gm = m0 + NT * orb + om;
  if (gm >= M || on >= N) return;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    if (bias) s[e] = __fadd_rn(s[e], bias[min(on + e, N - 1)]);
    if (relu) s[e] = fmaxf(0.0f, s[e]);
  }
  float* out = C + (int64_t)gm * ldc + on;
  if (on + 3 < N && ((reinterpret_cast<uintptr_t>(out) & 15) == 0)) {
    *reinterpret_cast<f32x4*>(out) = s;
  } else {
#pragma unroll
    for (int e = 0; e < 4; ++e)
      if (on + e < N) out[e] = s[e];
  }
}

template <int NB>
void launch_f32_narrow(cigemmContext* ctx, int64_t M, int64_t N, int64_t K, const float* A,
                       int64_t lda, const float* B, int64_t ldb, float* C, int64_t ldc,
                       const float* bias, bool relu) {
  // 16 rows per workgroup: many small workgroups spread evenly over the compute units (64
  // rows each left a quarter of them with twice the rows of the others: 16.4 against 13.0 us
  // for the 20000 x 512 x 10 layer)
  const dim3 grid((unsigned)((M + NT - 1) / NT)), block(256);
  // the waves' shares of a contiguous, aligned B pass through LDS when they fit 10 KiB each
  const size_t wave_bytes = (size_t)NB * 16 * (size_t)N * sizeof(float), stage_bytes = 4 * wave_bytes;
  const bool stage = ldb == N && (reinterpret_cast<uintptr_t>(B) & 15) == 0 && wave_bytes <= 10240;
  if (stage)
    hipLaunchKernelGGL((f32_narrow_kernel<NB, 1, true>), grid, block, stage_bytes, ctx->stream,
                       (int)M, (int)N, (int)K, A, lda, B, ldb, C, ldc, bias, relu ? 1 : 0);
  else
    hipLaunchKernelGGL((f32_narrow_kernel<NB, 1, false>), grid, block, 0, ctx->stream, (int)M,
                       (int)N, (int)K, A, lda, B, ldb, C, ldc, bias, relu ? 1 : 0);
}

}  // namespace

bool f32_small_shape_ok(int64_t M, int64_t N, int64_t K, const float* A, int64_t lda) {
  if (M <= 0 || N <= 0 || K <= 0 || K % 8) return false;
  if (lda % 4 || (reinterpret_cast<uintptr_t>(A) & 15)) return false;
  if (M > (1 << 24) || N > (1 << 24) || K > (1 << 24)) return false;
  const int64_t tiles = ((M + ST - 1) / ST) * ((N + ST - 1) / ST);
  return tiles <= 0x7fffffff;
}

void launch_f32_small(cigemmContext* ctx, int64_t M, int64_t N, int64_t K, const float* A,
                      int64_t lda, const float* B, int64_t ldb, float* C, int64_t ldc,
                      const BiasAct* ba) {
  const float* bias = ba ? ba->bias : nullptr;
  const bool relu = ba && ba->relu;
  // narrow outputs with a k share per wave that fits the registers
  const int64_t nb_wave = (K / 16 + 3) / 4;
  if (N <= NT && K % 16 == 0 && nb_wave <= 32 && M >= 64) {
    if (nb_wave <= 8)
      launch_f32_narrow<8>(ctx, M, N, K, A, lda, B, ldb, C, ldc, bias, relu);
    else if (nb_wave <= 16)
      launch_f32_narrow<16>(ctx, M, N, K, A, lda, B, ldb, C, ldc, bias, relu);
    else
      launch_f32_narrow<32>(ctx, M, N, K, A, lda, B, ldb, C, ldc, bias, relu);
    ctx->last_kernel = ba ? "f32_mfma_small_16x16_ksplit4_bias_act" : "f32_mfma_small_16x16_ksplit4";
    return;
  }
  const int tiles_m = (int)((M + ST - 1) / ST), tiles_n = (int)((N + ST - 1) / ST);
  const dim3 grid((unsigned)(tiles_m * (int64_t)tiles_n)), block(256);
  // 16-byte loads of B's rows: every quad of columns whole and aligned
  const bool bvec = N % 4 == 0 && ldb % 4 == 0 && (reinterpret_cast<uintptr_t>(B) & 15) == 0;
#define CIG_SMALL(HB, RL)                                                                        \
  do {                                                                                           \
    if (bvec)                                                                                    \
      hipLaunchKernelGGL((f32_small_kernel<HB, RL, true>), grid, block, 0, ctx->stream, (int)M,  \
                         (int)N, (int)K, tiles_n, A, lda, B, ldb, C, ldc, bias);                 \
    else                                                                                         \
      hipLaunchKernelGGL((f32_small_kernel<HB, RL, false>), grid, block, 0, ctx->stream, (int)M, \
                         (int)N, (int)K, tiles_n, A, lda, B, ldb, C, ldc, bias);                 \
  } while (0)
  if (bias) {
    if (relu) CIG_SMALL(true, true); else CIG_SMALL(true, false);
  } else {
    if (relu) CIG_SMALL(false, true); else CIG_SMALL(false, false);
  }
#undef CIG_SMALL
  ctx->last_kernel = ba ? "f32_mfma_small_32x32_ksplit4_bias_act" : "f32_mfma_small_32x32_ksplit4";
}

}  // namespace cig
