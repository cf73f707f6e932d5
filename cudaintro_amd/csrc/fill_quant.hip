// Device-side input generation and the absmax int8 quantizer.
//
// fill_random_*: the stateless hash generators of the reference's suite
// (quantization/GEMM_fp32.cu:7-17, GEMM_bf16.cu:8-19, GEMM_fp16.cu:8-19,
// GEMM_int8.cu:8-19).  Element idx depends only on (idx, seed), so the kernels are
// written as grid-stride loops over 16-byte stores: HBM-write bound.
//
// quantize_rows_i8: one workgroup per row, absmax then scale+round.  Rows of whole 16-byte
// pieces up to 16384 columns are held in registers between the two (read once, 16-byte
// loads, 4-byte stores); any other row is read twice, element by element.
#include "common.h"

namespace cig {
namespace {

constexpr uint64_t kHashMul = 2862933555777941757ULL, kHashAdd = 3037000493ULL;
__device__ __forceinline__ uint64_t hash64(int64_t idx, uint64_t seed) {
  uint64_t x = (uint64_t)idx ^ seed;
  return x * kHashMul + kHashAdd;
}

// n / 16777215.0f, correctly rounded, for an integer n below 2^24: the product with the
// rounded reciprocal plus one fused correction step.  Equal to the IEEE division for every one
// of the 2^24 numerators (checked exhaustively on the host, where fmaf is the same operation)
// at a third of its instructions.
__device__ __forceinline__ float div_by_16777215(float n) {
  const float d = 16777215.0f, rcp = 0x1.000002p-24f;  // rcp = fl(1 / d)
  const float q = __fmul_rn(n, rcp);
  return __fmaf_rn(__fmaf_rn(-q, d, n), rcp, q);
}

// The affine map is kept as separately rounded fp32 operations so the value equals the host
// formula bit for bit (no fusing).
__device__ __forceinline__ float hash_to_float(uint64_t x, float lo, float hi) {
  const float r = div_by_16777215((float)((x >> 11) & 0xFFFFFF));
  return __fadd_rn(lo, __fmul_rn(r, __fsub_rn(hi, lo)));
}

struct GenF32 {
  typedef float T;
  float lo, hi;
  __device__ __forceinline__ float operator()(uint64_t x) const { return hash_to_float(x, lo, hi); }
};
template <typename E16>
struct Gen16 {
  typedef uint16_t T;
  float lo, hi;
  __device__ __forceinline__ uint16_t operator()(uint64_t x) const {
    return E16::narrow(hash_to_float(x, lo, hi));
  }
};
// r % m for r < 2^16 and 1 <= m <= 256 without a division: q = (r * magic) >> 32 with
// magic = floor(2^32 / m) + 1 is floor(r / m) exactly for such r (m = 1, whose magic does not
// fit 32 bits, has remainder 0); checked exhaustively on the host.
struct GenI8 {
  typedef int8_t T;
  int lo;
  uint32_t m, magic;
  GenI8(int lo_, int hi_)
      : lo(lo_), m((uint32_t)(hi_ - lo_ + 1)),
        magic(m > 1 ? (uint32_t)((1ull << 32) / m) + 1u : 0u) {}
  __device__ __forceinline__ int8_t operator()(uint64_t x) const {
    const uint32_t r = (uint32_t)(x >> 11) & 0xFFFFu;
    const uint32_t rem = m > 1 ? r - __umulhi(r, magic) * m : 0u;
    return (int8_t)(lo + (int)rem);
  }
};

// Each lane produces 16 bytes (VEC elements) per step when the pointer is 16-byte aligned;
// the head (to alignment) and tail are written element-wise by the first lanes.
template <typename Gen>
__global__ __launch_bounds__(256) void fill_kernel(typename Gen::T* __restrict__ data,
                                                   int64_t count, uint64_t seed, Gen gen) {
  typedef typename Gen::T T;
  constexpr int VEC = 16 / sizeof(T);
  const int64_t tid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t nthreads = (int64_t)gridDim.x * blockDim.x;
  // elements before the first 16-byte boundary
  int64_t head = (int64_t)(((16 - ((uintptr_t)data & 15)) & 15) / sizeof(T));
  if (head > count) head = count;
  const int64_t nvec = (count - head) / VEC;
  if (head == 0) {
    // Aligned buffer: the VEC indices of a piece differ in their low bits only, so
    // (base + e) ^ seed = ((base ^ seed) & ~(VEC-1)) + ((seed ^ e) & (VEC-1)) and the hash is
    // one 64-bit multiply per piece plus, per element, the addition of a wave-uniform
    // multiple of the multiplier.
    uint64_t off[VEC];
#pragma unroll
    for (int e = 0; e < VEC; ++e) off[e] = ((seed ^ (uint64_t)e) & (VEC - 1)) * kHashMul;
    for (int64_t v = tid; v < nvec; v += nthreads) {
      const int64_t base = v * VEC;
      const uint64_t p = (((uint64_t)base ^ seed) & ~(uint64_t)(VEC - 1)) * kHashMul + kHashAdd;
      alignas(16) T tmp[VEC];
#pragma unroll
      for (int e = 0; e < VEC; ++e) tmp[e] = gen(p + off[e]);
      *reinterpret_cast<u32x4*>(data + base) = *reinterpret_cast<const u32x4*>(tmp);
    }
  } else {
    for (int64_t v = tid; v < nvec; v += nthreads) {
      const int64_t base = head + v * VEC;
      alignas(16) T tmp[VEC];
#pragma unroll
      for (int e = 0; e < VEC; ++e) tmp[e] = gen(hash64(base + e, seed));
      *reinterpret_cast<u32x4*>(data + base) = *reinterpret_cast<const u32x4*>(tmp);
    }
  }
  const int64_t tail0 = head + nvec * VEC;
  for (int64_t i = tid; i < head; i += nthreads) data[i] = gen(hash64(i, seed));
  for (int64_t i = tail0 + tid; i < count; i += nthreads) data[i] = gen(hash64(i, seed));
}

template <typename Gen>
void launch_fill(cigemmContext* ctx, typename Gen::T* data, int64_t count, uint64_t seed,
                 Gen gen) {
  constexpr int VEC = 16 / sizeof(typename Gen::T);
  int64_t blocks = (count / VEC + 255) / 256;
  const int64_t cap = (int64_t)ctx->num_cus * 16;
  if (blocks > cap) blocks = cap;
  if (blocks < 1) blocks = 1;
  hipLaunchKernelGGL((fill_kernel<Gen>), dim3((unsigned)blocks), dim3(256), 0, ctx->stream, data,
                     count, seed, gen);
}

__global__ __launch_bounds__(256) void quantize_rows_kernel(int64_t cols,
                                                            const float* __restrict__ x,
                                                            int64_t ldx, int8_t* __restrict__ q,
                                                            int64_t ldq,
                                                            float* __restrict__ scale) {
  __shared__ float red[4];
  const int64_t row = blockIdx.x;
  const float* xr = x + row * ldx;
  int8_t* qr = q + row * ldq;
  float amax = 0.0f;
  for (int64_t j = threadIdx.x; j < cols; j += 256) amax = fmaxf(amax, fabsf(xr[j]));
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off, 64));
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = amax;
  __syncthreads();
  amax = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
  const float s = amax > 0.0f ? __fdiv_rn(amax, 127.0f) : 1.0f;
  if (threadIdx.x == 0) scale[row] = s;
  for (int64_t j = threadIdx.x; j < cols; j += 256) {
    float r = rintf(__fdiv_rn(xr[j], s));  // ties to even
    r = fminf(fmaxf(r, -127.0f), 127.0f);
    qr[j] = (int8_t)(int)r;
  }
}

// The same for rows of whole 16-byte pieces (cols a multiple of 4, aligned rows) of up to
// 1024 * CHUNKS columns: a lane keeps its CHUNKS pieces of the row in registers, so the row is
// read once, as 16-byte loads, and written as packed 4-byte stores.  Same arithmetic per
// element as the kernel above (the maximum does not depend on the order it is taken in).
template <int CHUNKS>
__global__ __launch_bounds__(256) void quantize_rows_vec_kernel(int64_t cols,
                                                                const float* __restrict__ x,
                                                                int64_t ldx,
                                                                int8_t* __restrict__ q,
                                                                int64_t ldq,
                                                                float* __restrict__ scale) {
  __shared__ float red[4];
  const int64_t row = blockIdx.x;
  const f32x4* xr = reinterpret_cast<const f32x4*>(x + row * ldx);
  uint32_t* qr = reinterpret_cast<uint32_t*>(q + row * ldq);
  const int nquad = (int)(cols >> 2);
  f32x4 v[CHUNKS];
  float amax = 0.0f;
#pragma unroll
  for (int c = 0; c < CHUNKS; ++c) {
    const int i = threadIdx.x + 256 * c;
    v[c] = i < nquad ? xr[i] : f32x4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int e = 0; e < 4; ++e) amax = fmaxf(amax, fabsf(v[c][e]));
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off, 64));
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = amax;
  __syncthreads();
  amax = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
  const float s = amax > 0.0f ? __fdiv_rn(amax, 127.0f) : 1.0f;
  if (threadIdx.x == 0) scale[row] = s;
#pragma unroll
  for (int c = 0; c < CHUNKS; ++c) {
    const int i = threadIdx.x + 256 * c;
    uint32_t packed = 0;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      float r = rintf(__fdiv_rn(v[c][e], s));  // ties to even
      r = fminf(fmaxf(r, -127.0f), 127.0f);
      packed |= ((uint32_t)(int)r & 0xffu) << (8 * e);
    }
    if (i < nquad) qr[i] = packed;
  }
}

template <int CHUNKS>
void launch_quantize_vec(cigemmContext* ctx, int64_t rows, int64_t cols, const float* x,
                         int64_t ldx, int8_t* q, int64_t ldq, float* scale) {
  hipLaunchKernelGGL((quantize_rows_vec_kernel<CHUNKS>), dim3((unsigned)rows), dim3(256), 0,
                     ctx->stream, cols, x, ldx, q, ldq, scale);
}

}  // namespace
}  // namespace cig

using namespace cig;

static cigemmStatus_t fill_common(cigemmHandle_t h, const void* data, int64_t count,
                                  const char* name) {
  if (!h || h->magic != kCtxMagic) return CIGEMM_STATUS_NOT_INITIALIZED;
  if (count < 0) return fail(h, CIGEMM_STATUS_INVALID_VALUE, "%s: count %lld < 0", name,
                             (long long)count);
  if (count > 0 && !data) return fail(h, CIGEMM_STATUS_INVALID_VALUE, "%s: null data", name);
  return CIGEMM_STATUS_SUCCESS;
}

extern "C" {

cigemmStatus_t cigemm_fill_random_f32(cigemmHandle_t h, float* data, int64_t count,
                                      uint64_t seed, float lo, float hi) {
  cigemmStatus_t st = fill_common(h, data, count, "cigemm_fill_random_f32");
  if (st != CIGEMM_STATUS_SUCCESS || count == 0) return st;
  launch_fill(h, data, count, seed, GenF32{lo, hi});
  return check_launch(h, "cigemm_fill_random_f32");
}

cigemmStatus_t cigemm_fill_random_bf16(cigemmHandle_t h, uint16_t* data, int64_t count,
                                       uint64_t seed, float lo, float hi) {
  cigemmStatus_t st = fill_common(h, data, count, "cigemm_fill_random_bf16");
  if (st != CIGEMM_STATUS_SUCCESS || count == 0) return st;
  launch_fill(h, data, count, seed, Gen16<BF16>{lo, hi});
  return check_launch(h, "cigemm_fill_random_bf16");
}

cigemmStatus_t cigemm_fill_random_f16(cigemmHandle_t h, uint16_t* data, int64_t count,
                                      uint64_t seed, float lo, float hi) {
  cigemmStatus_t st = fill_common(h, data, count, "cigemm_fill_random_f16");
  if (st != CIGEMM_STATUS_SUCCESS || count == 0) return st;
  launch_fill(h, data, count, seed, Gen16<F16>{lo, hi});
  return check_launch(h, "cigemm_fill_random_f16");
}

cigemmStatus_t cigemm_fill_random_i8(cigemmHandle_t h, int8_t* data, int64_t count,
                                     uint64_t seed, int lo, int hi) {
  cigemmStatus_t st = fill_common(h, data, count, "cigemm_fill_random_i8");
  if (st != CIGEMM_STATUS_SUCCESS) return st;
  if (hi < lo || lo < -128 || hi > 127)
    return fail(h, CIGEMM_STATUS_INVALID_VALUE, "cigemm_fill_random_i8: bad range [%d,%d]", lo, hi);
  if (count == 0) return st;
  launch_fill(h, data, count, seed, GenI8(lo, hi));
  return check_launch(h, "cigemm_fill_random_i8");
}

cigemmStatus_t cigemm_quantize_rows_i8(cigemmHandle_t h, int64_t rows, int64_t cols,
                                       const float* x, int64_t ldx, int8_t* q, int64_t ldq,
                                       float* scale) {
  if (!h || h->magic != kCtxMagic) return CIGEMM_STATUS_NOT_INITIALIZED;
  if (rows < 0 || cols < 0)
    return fail(h, CIGEMM_STATUS_INVALID_VALUE, "cigemm_quantize_rows_i8: negative size");
  if (rows == 0) return CIGEMM_STATUS_SUCCESS;
  if (!scale || (cols > 0 && (!x || !q)))
    return fail(h, CIGEMM_STATUS_INVALID_VALUE, "cigemm_quantize_rows_i8: null pointer");
  if (ldx < cols || ldq < cols)
    return fail(h, CIGEMM_STATUS_INVALID_VALUE, "cigemm_quantize_rows_i8: ld < cols");
  if (rows > 2147483647LL)
    return fail(h, CIGEMM_STATUS_NOT_SUPPORTED, "cigemm_quantize_rows_i8: rows > 2^31-1");
  const bool pieces = cols > 0 && cols % 4 == 0 && ldx % 4 == 0 && ldq % 4 == 0 &&
                      ((uintptr_t)x & 15) == 0 && ((uintptr_t)q & 3) == 0 && cols <= 16384;
  if (pieces && cols <= 1024)
    launch_quantize_vec<1>(h, rows, cols, x, ldx, q, ldq, scale);
  else if (pieces && cols <= 2048)
    launch_quantize_vec<2>(h, rows, cols, x, ldx, q, ldq, scale);
  else if (pieces && cols <= 4096)
    launch_quantize_vec<4>(h, rows, cols, x, ldx, q, ldq, scale);
  else if (pieces && cols <= 8192)
    launch_quantize_vec<8>(h, rows, cols, x, ldx, q, ldq, scale);
  else if (pieces)
    launch_quantize_vec<16>(h, rows, cols, x, ldx, q, ldq, scale);
  else
    hipLaunchKernelGGL(quantize_rows_kernel, dim3((unsigned)rows), dim3(256), 0, h->stream, cols,
                       x, ldx, q, ldq, scale);
  return check_launch(h, "cigemm_quantize_rows_i8");
}

}  // extern "C"
