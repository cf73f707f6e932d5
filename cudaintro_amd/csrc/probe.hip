// Measurement aid: a register-resident matrix-core loop (no memory traffic in the loop), one
// wave per SIMD on every compute unit, to show what the chip sustains at the clock it
// actually holds under this load.  Sustained rate depends on the operand data (the chip is
// power limited), so the probe runs on constant or on pseudo-random operand bits.
#include <algorithm>
#include <type_traits>
#include <vector>

#include "cigemm_probe.h"
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


// ---- what the other instructions of the tile kernel's main loop cost ---------------------
// One "stage" = two k-steps of 16 bf16 32x32x16 matrix instructions on a 4 x 4 grid of
// accumulator tiles (the 128 x 128 wave tile of the product kernel), fragments double buffered
// in registers.  Optional, at the places the product kernel's schedule puts them: 12 LDS
// fragment reads per k-step (4 of 16 bytes, 8 transposing ones of 8 bytes) for the other
// fragment buffer, NDMA LDS-DMA instructions in the second k-step, one wait and one workgroup
// barrier between the k-steps.  Every slot (one matrix instruction, at most one read, at most
// one DMA) is closed by a scheduling fence.
typedef __attribute__((address_space(3))) i16x4 probe_lds_i16x4;

// Where the DMA instructions go: instruction d of wave w sits in slot (w * WOFF + d * STRIDE)
// mod 32 of the 32 slots between one barrier and the next (slots 0..15: the k-step after the
// barrier, 16..31: the k-step before the next one).  STRIDE 1, WOFF 0 is the product kernel's
// placement before it was spread: every wave issues its instructions back to back right after
// the barrier, so that the compute unit's one address path sees all of them at once.
constexpr bool dma_in_slot(int g, int off, int stride, int ndma) {
  for (int d = 0; d < ndma; ++d)
    if ((off + d * stride) % 32 == g) return true;
  return false;
}
constexpr int dma_index(int g, int off, int stride, int ndma) {
  for (int d = 0; d < ndma; ++d)
    if ((off + d * stride) % 32 == g) return d;
  return 0;
}

template <int NDMA, int NLDS, int BARRIER, int STRIDE, int WOFF, int MFMA>
__global__ __launch_bounds__(256, 1) void issue_cost_kernel(const char* __restrict__ src,
                                                            uint64_t* __restrict__ stamps,
                                                            float* __restrict__ sink, int iters,
                                                            int src_span) {
  extern __shared__ __attribute__((aligned(1024))) char lds[];
  const int t = threadIdx.x, l = t & 63;
  const int w = __builtin_amdgcn_readfirstlane(t >> 6);
  // per wave: 8 KiB that the fragment reads read, 8 KiB that the DMA fills and nothing reads
  char* rd = lds + w * 16384;
  const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)lds;
  const uint32_t dma_dst = lds_base + w * 16384 + 8192;
  for (int i = l * 16; i < 8192; i += 1024) {
    u32x4 v;
#pragma unroll
    for (int e = 0; e < 4; ++e)  // +-[1,2) in bf16, pseudo-random sign and mantissa
      v[e] = (mix32((uint32_t)(blockIdx.x * 65536 + w * 8192 + i + e + 1)) & 0x807f807fu) | 0x3f803f80u;
    *reinterpret_cast<u32x4*>(rd + i) = v;
  }
  __syncthreads();
  // the wave's DMA source: `src_span` bytes walked 8 KiB per stage, round and round (8 KiB: the
  // same lines every stage, served by the vector L1; more than the L1 holds: by the L2)
  const char* const my_src0 = src + ((size_t)blockIdx.x * 4 + w) * (size_t)src_span;
  const char* my_src = my_src0;
  int src_off = 0;
  const uint32_t voff = (uint32_t)l * 16;
  struct Frags {
    u32x4 a[4];
    u32x2 b[8];
  };
  auto read_piece = [&](Frags& f, int kk, int r) {
    if (r < 4)
      f.a[r] = *reinterpret_cast<const u32x4*>(rd + (r ^ kk) * 1024 + l * 16);
    else
      f.b[r - 4] = __builtin_bit_cast(
          u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                     (probe_lds_i16x4*)(rd + 4096 + ((r - 4) ^ kk) * 512 + l * 8)));
  };
  Frags f0, f1;
#pragma unroll
  for (int r = 0; r < 12; ++r) read_piece(f0, 0, r);
#pragma unroll
  for (int r = 0; r < 12; ++r) read_piece(f1, 1, r);
  f32x16 acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;
  uint32_t fold = 0;  // without matrix instructions: what consumes the fragments instead
  auto mfma_piece = [&](const Frags& f, int m) {
    if (!MFMA) {
      if (m == 15 && NLDS) {
#pragma unroll
        for (int r = 0; r < 4; ++r) fold ^= f.a[r][0];
#pragma unroll
        for (int r = 0; r < 8; ++r) fold ^= f.b[r][0];
      }
      return;
    }
    const int j = m / 4;
    const int i = (j & 1) ? 3 - m % 4 : m % 4;
    const u32x4 bfrag = __builtin_shufflevector(f.b[2 * j], f.b[2 * j + 1], 0, 1, 2, 3);
    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, bfrag),
                                                        __builtin_bit_cast(bf16x8, f.a[i]),
                                                        acc[i][j], 0, 0, 0);
  };
  auto dma = [&](int d) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :
                 : "s"(dma_dst + d * 1024), "v"(voff), "s"(my_src)
                 : "m0");
  };
  uint64_t t0 = 0, r0 = 0;
  if (l == 0) {
    t0 = __builtin_amdgcn_s_memtime();
    r0 = __builtin_amdgcn_s_memrealtime();
  }
  auto run = [&](auto off_const) {
    constexpr int OFF = decltype(off_const)::value;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int sl = 0; sl < 16; ++sl) {
        mfma_piece(f0, sl);
        if (NLDS && sl < 12) read_piece(f1, 1, sl);
        if (dma_in_slot(16 + sl, OFF, STRIDE, NDMA)) dma(dma_index(16 + sl, OFF, STRIDE, NDMA));
        if (sl == 13) {
          // the next stage's DMA source, computed here, in a slot that holds nothing else (a
          // lone wave issues one instruction per four cycles, and only about seven of them fit
          // under one matrix instruction: at the end of the loop, beside the branch, these few
          // scalar instructions would cost 24 cycles per stage)
          src_off = src_off + 8192 < src_span ? src_off + 8192 : 0;
          my_src = my_src0 + src_off;
        }
        __builtin_amdgcn_sched_barrier(0);
      }
      // (as in the product: everything but the DMA of the last two stages has landed)
      if (NDMA) __builtin_amdgcn_s_waitcnt(0x0f70 | ((2 * NDMA) & 15) | (((2 * NDMA) >> 4) << 14));
      if (BARRIER) __builtin_amdgcn_s_barrier();
      asm volatile("" ::: "memory");
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int sl = 0; sl < 16; ++sl) {
        mfma_piece(f1, sl);
        if (NLDS && sl < 12) read_piece(f0, 0, sl);
        if (dma_in_slot(sl, OFF, STRIDE, NDMA)) dma(dma_index(sl, OFF, STRIDE, NDMA));
        __builtin_amdgcn_sched_barrier(0);
      }
      asm volatile("" ::: "memory");
    }
  };
  if (WOFF == 0 || w == 0)
    run(std::integral_constant<int, 0>{});
  else if (w == 1)
    run(std::integral_constant<int, WOFF>{});
  else if (w == 2)
    run(std::integral_constant<int, 2 * WOFF>{});
  else
    run(std::integral_constant<int, 3 * WOFF>{});
  if (l == 0) {
    uint64_t* p = stamps + ((size_t)blockIdx.x * 4 + w) * 4;
    p[0] = t0;
    p[1] = __builtin_amdgcn_s_memtime();
    p[2] = r0;
    p[3] = __builtin_amdgcn_s_memrealtime();
  }
  __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): no DMA outlives the wave
  float sum = 0.0f;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) sum += acc[i][j][e];
  sink[blockIdx.x * 256 + t] = sum + (float)(fold & 1);
}

// Microseconds per tick of the constant-rate counter s_memrealtime reads.
double wall_tick_us(int device) {
  int khz = 0;
  if (hipDeviceGetAttribute(&khz, hipDeviceAttributeWallClockRate, device) != hipSuccess || khz <= 0) {
    (void)hipGetLastError();
    return 0.01;  // 100 MHz, gfx950's rate
  }
  return 1.0e3 / (double)khz;
}

constexpr int ISSUE_LDS_BYTES = 4 * 16384;

template <int NDMA, int NLDS, int BARRIER, int STRIDE = 1, int WOFF = 0, int MFMA = 1>
void launch_issue_cost(cigemmContext* ctx, int grid, const char* src, uint64_t* stamps, float* sink,
                       int iters, int src_span) {
  auto kern = issue_cost_kernel<NDMA, NLDS, BARRIER, STRIDE, WOFF, MFMA>;
  static std::atomic<uint64_t> lds_set{0};
  if (!ensure_dynamic_lds(ctx, (const void*)kern, ISSUE_LDS_BYTES, lds_set)) return;
  hipLaunchKernelGGL(kern, dim3(grid), dim3(256), ISSUE_LDS_BYTES, ctx->stream, src, stamps, sink,
                     iters, src_span);
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

extern "C" cigemmStatus_t cigemm_probe_issue_cost(cigemmHandle_t h, int n_dma, int n_lds_reads,
                                                  int barrier, int placement, int mfma,
                                                  int src_kib_per_wave, int workgroups, int iters,
                                                  double* result) {
  const char* name = "cigemm_probe_issue_cost";
  if (!h || h->magic != kCtxMagic) return CIGEMM_STATUS_NOT_INITIALIZED;
  const int cus = h->num_cus > 0 ? h->num_cus : 256;
  if ((n_dma != 0 && n_dma != 2 && n_dma != 4 && n_dma != 8) ||
      (n_lds_reads != 0 && n_lds_reads != 24) || (barrier != 0 && barrier != 1) || placement < 0 ||
      placement > 7 || (placement > 0 && (n_dma != 8 || (mfma && n_lds_reads != 24))) ||
      (mfma != 0 && mfma != 1) ||
      (!mfma && (placement > 1 || (n_dma != 0 && n_dma != 8))) || src_kib_per_wave < 8 ||
      src_kib_per_wave % 8 || src_kib_per_wave > 1024 || workgroups < 1 ||
      workgroups > cus || iters <= 0 || iters > (1 << 22) || !result)
    return fail(h, CIGEMM_STATUS_INVALID_VALUE,
                "%s: n_dma %d (0, 2, 4, 8), n_lds_reads %d (0, 24), barrier %d, placement %d (0..7; "
                "above 0 only with n_dma 8 and n_lds_reads 24), mfma %d (0 only with placement 0 or 1 "
                "and n_dma 0 or 8), src_kib_per_wave %d (8..1024, multiple of 8), workgroups %d "
                "(1..%d), iters %d",
                name, n_dma, n_lds_reads, barrier, placement, mfma, src_kib_per_wave, workgroups, cus,
                iters);
  // workspace: stamps (32 bytes per wave), the sink, then the DMA source of every wave
  const int src_span = src_kib_per_wave * 1024;
  const size_t stamp_bytes = (size_t)workgroups * 4 * 32, sink_bytes = (size_t)workgroups * 1024;
  const size_t src_off = (stamp_bytes + sink_bytes + 4095) & ~(size_t)4095;
  if (!h->workspace || src_off + (size_t)workgroups * 4 * (size_t)src_span > h->ws_partial_bytes)
    return fail(h, CIGEMM_STATUS_NOT_SUPPORTED,
                "%s: %d workgroups x 4 waves x %d KiB of DMA source exceed the workspace", name,
                workgroups, src_kib_per_wave);
  char* ws = static_cast<char*>(h->workspace);
  uint64_t* stamps = reinterpret_cast<uint64_t*>(ws);
  float* sink = reinterpret_cast<float*>(ws + stamp_bytes);
  const char* src = ws + src_off;
#define CIG_IC(D, L, B) launch_issue_cost<D, L, B>(h, workgroups, src, stamps, sink, iters, src_span)
#define CIG_IC_B(D, L) do { if (barrier) CIG_IC(D, L, 1); else CIG_IC(D, L, 0); } while (0)
#define CIG_IC_L(D) do { if (n_lds_reads) CIG_IC_B(D, 24); else CIG_IC_B(D, 0); } while (0)
#define CIG_IC_P(S, W)                                                                   \
  do {                                                                                   \
    if (barrier)                                                                         \
      launch_issue_cost<8, 24, 1, S, W>(h, workgroups, src, stamps, sink, iters, src_span); \
    else                                                                                 \
      launch_issue_cost<8, 24, 0, S, W>(h, workgroups, src, stamps, sink, iters, src_span); \
  } while (0)
#define CIG_IC_N(D, L, S)                                                                        \
  do {                                                                                           \
    if (barrier)                                                                                 \
      launch_issue_cost<D, L, 1, S, 0, 0>(h, workgroups, src, stamps, sink, iters, src_span);    \
    else                                                                                         \
      launch_issue_cost<D, L, 0, S, 0, 0>(h, workgroups, src, stamps, sink, iters, src_span);    \
  } while (0)
  if (!mfma) {  // the stage's memory instructions alone, 32-cycle slots left empty
    if (n_dma == 8 && n_lds_reads) {
      if (placement) CIG_IC_N(8, 24, 2); else CIG_IC_N(8, 24, 1);
    } else if (n_dma == 8) {
      if (placement) CIG_IC_N(8, 0, 2); else CIG_IC_N(8, 0, 1);
    } else if (n_lds_reads) {
      CIG_IC_N(0, 24, 1);
    } else {
      CIG_IC_N(0, 0, 1);
    }
  } else
  switch (placement) {
    case 1: CIG_IC_P(2, 0); break;   // every second slot of the k-step after the barrier
    case 2: CIG_IC_P(2, 1); break;   // ... waves 1 and 3 on the odd slots
    case 3: CIG_IC_P(4, 0); break;   // every fourth slot, over both k-steps
    case 4: CIG_IC_P(4, 1); break;   // ... wave w one slot after wave w - 1
    case 5: CIG_IC_P(1, 4); break;   // back to back, wave w four slots after wave w - 1
    case 6: CIG_IC_P(1, 8); break;   // back to back, wave w eight slots after wave w - 1
    case 7: CIG_IC_P(2, 8); break;   // every second slot, wave w eight slots after wave w - 1
    default:
      switch (n_dma) {
        case 0: CIG_IC_L(0); break;
        case 2: CIG_IC_L(2); break;
        case 4: CIG_IC_L(4); break;
        default: CIG_IC_L(8); break;
      }
  }
#undef CIG_IC_P
#undef CIG_IC_N
#undef CIG_IC_L
#undef CIG_IC_B
#undef CIG_IC
  cigemmStatus_t st = check_launch(h, name);
  if (st != CIGEMM_STATUS_SUCCESS) return st;
  std::vector<uint64_t> host((size_t)workgroups * 16);
  if (hipMemcpyAsync(host.data(), stamps, host.size() * 8, hipMemcpyDeviceToHost, h->stream) != hipSuccess ||
      hipStreamSynchronize(h->stream) != hipSuccess) {
    (void)hipGetLastError();
    h->ws_dirty = 1;
    return fail(h, CIGEMM_STATUS_EXECUTION_FAILED, "%s: reading the stamps back failed", name);
  }
  const double tick_us = wall_tick_us(h->device);
  double cycles = 0, worst = 0, ticks = 0;
  uint64_t first = ~0ull, last = 0;
  for (int i = 0; i < workgroups * 4; ++i) {
    const uint64_t* p = &host[(size_t)i * 4];
    const double c = (double)(p[1] - p[0]);
    cycles += c;
    worst = std::max(worst, c);
    ticks += (double)(p[3] - p[2]);
    first = std::min(first, p[2]);
    last = std::max(last, p[3]);
  }
  result[0] = cycles / (workgroups * 4) / iters;
  result[1] = worst / iters;
  result[2] = ticks > 0 ? cycles / (ticks * tick_us) * 1e-3 : 0.0;
  result[3] = (double)(last - first) * tick_us;
  h->last_kernel = "issue_cost_probe";
  return CIGEMM_STATUS_SUCCESS;
}

extern "C" cigemmStatus_t cigemm_probe_dirty_workspace(cigemmHandle_t h, int count, uint32_t value,
                                                       int mark_dirty) {
  const char* name = "cigemm_probe_dirty_workspace";
  if (!h || h->magic != kCtxMagic) return CIGEMM_STATUS_NOT_INITIALIZED;
  if (count < 0 || (size_t)count * 4 > h->ws_counter_bytes || (size_t)count * 8 > h->ws_swap_bytes ||
      !h->workspace)
    return fail(h, CIGEMM_STATUS_INVALID_VALUE, "%s: count %d", name, count);
  if (count > 0) {
    char* base = static_cast<char*>(h->workspace) + h->ws_partial_bytes;
    std::vector<uint32_t> c32((size_t)count, value);
    std::vector<uint64_t> c64((size_t)count, ((uint64_t)value << 32) | value);
    if (hipMemcpyAsync(base, c32.data(), c32.size() * 4, hipMemcpyHostToDevice, h->stream) != hipSuccess ||
        hipMemcpyAsync(base + h->ws_counter_bytes, c64.data(), c64.size() * 8, hipMemcpyHostToDevice,
                       h->stream) != hipSuccess ||
        hipStreamSynchronize(h->stream) != hipSuccess) {
      (void)hipGetLastError();
      return fail(h, CIGEMM_STATUS_EXECUTION_FAILED, "%s: copy failed", name);
    }
  }
  if (mark_dirty) h->ws_dirty = 1;
  return CIGEMM_STATUS_SUCCESS;
}

extern "C" cigemmStatus_t cigemm_probe_force_tile_plan(cigemmHandle_t h, int tile_rows,
                                                       int k_ranges) {
  const char* name = "cigemm_probe_force_tile_plan";
  if (!h || h->magic != kCtxMagic) return CIGEMM_STATUS_NOT_INITIALIZED;
  if (tile_rows == 0) {
    h->force_tile_mt = h->force_tile_splits = 0;
    return CIGEMM_STATUS_SUCCESS;
  }
  if (tile_rows % 64 || tile_rows < 64 || tile_rows > 256 || k_ranges < 1 || k_ranges > 64)
    return fail(h, CIGEMM_STATUS_INVALID_VALUE, "%s: tile_rows %d, k_ranges %d", name, tile_rows,
                k_ranges);
  h->force_tile_mt = tile_rows / 64;
  h->force_tile_splits = k_ranges;
  return CIGEMM_STATUS_SUCCESS;
}
