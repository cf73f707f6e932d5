// C ABI: handle lifecycle, argument validation and dispatch to the kernel families.
// Validation happens entirely on the host, before any launch: a call that returns a
// non-success status has enqueued nothing.
#include <cstdlib>
#include <new>

#include "common.h"

namespace cig {
namespace {

bool valid(cigemmHandle_t h) { return h && h->magic == kCtxMagic; }

// Common checks of one C[MxN] = A[MxK] . B GEMM call.  b_rows x b_cols is B's stored shape.
cigemmStatus_t check_gemm_args(cigemmHandle_t h, const char* name, int64_t M, int64_t N,
                               int64_t K, const void* A, int64_t lda, const void* B,
                               int64_t ldb, int64_t b_cols, const void* C, int64_t ldc) {
  h->last_tile_rows = 0;  // set again by the tile kernel's launcher
  h->last_k_splits = 0;
  h->last_waves = 0;
  h->last_per_cu = 1;
  h->first_tile_rows = 0;
  h->first_waves = 0;
  if (h->ws_dirty) clear_workspace(h);  // a call before this one ended in EXECUTION_FAILED
  if (M < 0 || N < 0 || K < 0)
    return fail(h, CIGEMM_STATUS_INVALID_VALUE, "%s: negative dimension (M=%lld N=%lld K=%lld)",
                name, (long long)M, (long long)N, (long long)K);
  if (M == 0 || N == 0) return CIGEMM_STATUS_SUCCESS;
  if (!C) return fail(h, CIGEMM_STATUS_INVALID_VALUE, "%s: null output pointer", name);
  if (ldc < N)
    return fail(h, CIGEMM_STATUS_INVALID_VALUE, "%s: ldc=%lld < N=%lld", name, (long long)ldc,
                (long long)N);
  if (K > 0) {
    if (!A || !B) return fail(h, CIGEMM_STATUS_INVALID_VALUE, "%s: null input pointer", name);
    if (lda < K)
      return fail(h, CIGEMM_STATUS_INVALID_VALUE, "%s: lda=%lld < K=%lld", name, (long long)lda,
                  (long long)K);
    if (ldb < b_cols)
      return fail(h, CIGEMM_STATUS_INVALID_VALUE, "%s: ldb=%lld < %lld", name, (long long)ldb,
                  (long long)b_cols);
  }
  if ((M + 63) / 64 > 65535)
    return fail(h, CIGEMM_STATUS_NOT_SUPPORTED, "%s: M=%lld exceeds the launch grid", name,
                (long long)M);
  if (K > 2147483647LL || N > 2147483647LL)
    return fail(h, CIGEMM_STATUS_NOT_SUPPORTED, "%s: N or K exceeds 2^31-1", name);
  return CIGEMM_STATUS_SUCCESS;
}

}  // namespace
}  // namespace cig

using namespace cig;

extern "C" {

cigemmStatus_t cigemmCreate(cigemmHandle_t* handle) {
  if (!handle) return CIGEMM_STATUS_INVALID_VALUE;
  *handle = nullptr;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) {
    (void)hipGetLastError();
    return CIGEMM_STATUS_NOT_INITIALIZED;
  }
  hipDeviceProp_t prop;
  if (hipGetDeviceProperties(&prop, dev) != hipSuccess) {
    (void)hipGetLastError();
    return CIGEMM_STATUS_NOT_INITIALIZED;
  }
  if (strncmp(prop.gcnArchName, "gfx950", 6) != 0) return CIGEMM_STATUS_ARCH_MISMATCH;
  cigemmContext* ctx = new (std::nothrow) cigemmContext();
  if (!ctx) return CIGEMM_STATUS_ALLOC_FAILED;
  ctx->magic = kCtxMagic;
  ctx->device = dev;
  ctx->num_cus = prop.multiProcessorCount;
  ctx->stream = nullptr;
  ctx->last_kernel = "";
  ctx->last_tile_rows = 0;
  ctx->last_k_splits = 0;
  ctx->last_waves = 0;
  ctx->last_per_cu = 1;
  ctx->first_tile_rows = 0;
  ctx->first_waves = 0;
  ctx->kernel_name[0] = '\0';
  ctx->pending_error[0] = '\0';
  ctx->algo = CIGEMM_ALGO_DEFAULT;
  ctx->last_error[0] = '\0';
  ctx->ws_partial_bytes = (size_t)64 << 20;
  ctx->ws_counter_bytes = (size_t)64 << 10;
  ctx->ws_swap_bytes = (size_t)8 << 20;  // 128 bytes per column: N <= 65536
  ctx->ws_dirty = 0;
  ctx->force_tile_mt = 0;
  ctx->force_tile_splits = 0;
  ctx->workspace = nullptr;
  if (hipMalloc(&ctx->workspace,
                ctx->ws_partial_bytes + ctx->ws_counter_bytes + ctx->ws_swap_bytes) != hipSuccess ||
      hipMemset(static_cast<char*>(ctx->workspace) + ctx->ws_partial_bytes, 0,
                ctx->ws_counter_bytes + ctx->ws_swap_bytes) != hipSuccess) {
    (void)hipGetLastError();
    if (ctx->workspace) (void)hipFree(ctx->workspace);
    delete ctx;
    return CIGEMM_STATUS_ALLOC_FAILED;
  }
  *handle = ctx;
  return CIGEMM_STATUS_SUCCESS;
}

cigemmStatus_t cigemmDestroy(cigemmHandle_t h) {
  if (!valid(h)) return CIGEMM_STATUS_NOT_INITIALIZED;
  h->magic = 0;
  if (h->workspace) (void)hipFree(h->workspace);
  delete h;
  return CIGEMM_STATUS_SUCCESS;
}

cigemmStatus_t cigemmSetStream(cigemmHandle_t h, void* stream) {
  if (!valid(h)) return CIGEMM_STATUS_NOT_INITIALIZED;
  h->stream = static_cast<hipStream_t>(stream);
  return CIGEMM_STATUS_SUCCESS;
}

cigemmStatus_t cigemmResetWorkspace(cigemmHandle_t h) {
  if (!valid(h)) return CIGEMM_STATUS_NOT_INITIALIZED;
  clear_workspace(h);
  return check_launch(h, "cigemmResetWorkspace");
}

cigemmStatus_t cigemmGetStream(cigemmHandle_t h, void** stream) {
  if (!valid(h)) return CIGEMM_STATUS_NOT_INITIALIZED;
  if (!stream) return fail(h, CIGEMM_STATUS_INVALID_VALUE, "cigemmGetStream: null argument");
  *stream = h->stream;
  return CIGEMM_STATUS_SUCCESS;
}

const char* cigemmGetStatusString(cigemmStatus_t status) {
  switch (status) {
    case CIGEMM_STATUS_SUCCESS: return "CIGEMM_STATUS_SUCCESS";
    case CIGEMM_STATUS_NOT_INITIALIZED: return "CIGEMM_STATUS_NOT_INITIALIZED";
    case CIGEMM_STATUS_ALLOC_FAILED: return "CIGEMM_STATUS_ALLOC_FAILED";
    case CIGEMM_STATUS_INVALID_VALUE: return "CIGEMM_STATUS_INVALID_VALUE";
    case CIGEMM_STATUS_ARCH_MISMATCH: return "CIGEMM_STATUS_ARCH_MISMATCH";
    case CIGEMM_STATUS_MAPPING_ERROR: return "CIGEMM_STATUS_MAPPING_ERROR";
    case CIGEMM_STATUS_EXECUTION_FAILED: return "CIGEMM_STATUS_EXECUTION_FAILED";
    case CIGEMM_STATUS_INTERNAL_ERROR: return "CIGEMM_STATUS_INTERNAL_ERROR";
    case CIGEMM_STATUS_NOT_SUPPORTED: return "CIGEMM_STATUS_NOT_SUPPORTED";
    case CIGEMM_STATUS_LICENSE_ERROR: return "CIGEMM_STATUS_LICENSE_ERROR";
    default: return "CIGEMM_STATUS_UNKNOWN";
  }
}

const char* cigemmGetLastErrorString(cigemmHandle_t h) { return valid(h) ? h->last_error : ""; }

int cigemmGetVersion(void) { return 100; }

const char* cigemmGetLastKernelName(cigemmHandle_t h) { return valid(h) ? h->last_kernel : ""; }

cigemmStatus_t cigemmGetLastPlan(cigemmHandle_t h, int* tile_rows, int* k_splits) {
  if (!valid(h)) return CIGEMM_STATUS_NOT_INITIALIZED;
  if (tile_rows) *tile_rows = h->last_tile_rows;
  if (k_splits) *k_splits = h->last_k_splits;
  return CIGEMM_STATUS_SUCCESS;
}

cigemmStatus_t cigemmSetAlgo(cigemmHandle_t h, cigemmAlgo_t algo) {
  if (!valid(h)) return CIGEMM_STATUS_NOT_INITIALIZED;
  if ((int)algo < CIGEMM_ALGO_DEFAULT || (int)algo > CIGEMM_ALGO_MFMA_ANY)
    return fail(h, CIGEMM_STATUS_INVALID_VALUE, "cigemmSetAlgo: bad algo %d", (int)algo);
  h->algo = (int)algo;
  return CIGEMM_STATUS_SUCCESS;
}

cigemmStatus_t cigemmGetAlgo(cigemmHandle_t h, cigemmAlgo_t* algo) {
  if (!valid(h)) return CIGEMM_STATUS_NOT_INITIALIZED;
  if (!algo) return fail(h, CIGEMM_STATUS_INVALID_VALUE, "cigemmGetAlgo: null pointer");
  *algo = (cigemmAlgo_t)h->algo;
  return CIGEMM_STATUS_SUCCESS;
}

static cigemmStatus_t algo_refused(cigemmHandle_t h, const char* name) {
  return fail(h, CIGEMM_STATUS_NOT_SUPPORTED,
              "%s: the selected kernel family (algo %d) does not take this call", name, h->algo);
}

// fp32 dispatch.  DEFAULT: one of the two aligned MFMA kernels when the shape allows, else the
// any-shape MFMA kernel (the scalar kernel only if its tile grid does not fit a launch).
// Returns false when a selected family refuses the call.
static bool dispatch_f32(cigemmHandle_t h, int64_t M, int64_t N, int64_t K, const float* A,
                         int64_t lda, const float* B, int64_t ldb, float* C, int64_t ldc,
                         const BiasAct* ba) {
  switch (h->algo) {
    case CIGEMM_ALGO_TILE:
      return launch_f32_tile(h, M, N, K, A, lda, B, ldb, C, ldc, ba);
    case CIGEMM_ALGO_SMALL:
      if (!f32_small_shape_ok(M, N, K, A, lda)) return false;
      launch_f32_small(h, M, N, K, A, lda, B, ldb, C, ldc, ba);
      return true;
    case CIGEMM_ALGO_SKINNY:
      return false;
    case CIGEMM_ALGO_MFMA_ANY:
      return launch_mfma_any_f32(h, M, N, K, A, lda, B, ldb, C, ldc, ba);
    case CIGEMM_ALGO_GENERIC:
      launch_generic_f32(h, M, N, K, A, lda, B, ldb, C, ldc, ba);
      return true;
    default:
      if (!launch_f32_mfma(h, M, N, K, A, lda, B, ldb, C, ldc, ba) &&
          !launch_mfma_any_f32(h, M, N, K, A, lda, B, ldb, C, ldc, ba))
        launch_generic_f32(h, M, N, K, A, lda, B, ldb, C, ldc, ba);
      return true;
  }
}

cigemmStatus_t cigemm_gemm_f32(cigemmHandle_t h, int64_t M, int64_t N, int64_t K, const float* A,
                               int64_t lda, const float* B, int64_t ldb, float* C, int64_t ldc) {
  if (!valid(h)) return CIGEMM_STATUS_NOT_INITIALIZED;
  cigemmStatus_t st = check_gemm_args(h, "cigemm_gemm_f32", M, N, K, A, lda, B, ldb, N, C, ldc);
  if (st != CIGEMM_STATUS_SUCCESS || M == 0 || N == 0) return st;
  if (!dispatch_f32(h, M, N, K, A, lda, B, ldb, C, ldc, nullptr))
    return algo_refused(h, "cigemm_gemm_f32");
  return check_launch(h, "cigemm_gemm_f32");
}

cigemmStatus_t cigemm_linear_f32(cigemmHandle_t h, int64_t M, int64_t N, int64_t K, const float* X,
                                 int64_t ldx, const float* W, int64_t ldw, const float* bias,
                                 cigemmActivation_t act, float* out, int64_t ldo) {
  if (!valid(h)) return CIGEMM_STATUS_NOT_INITIALIZED;
  if (act != CIGEMM_ACT_NONE && act != CIGEMM_ACT_RELU)
    return fail(h, CIGEMM_STATUS_INVALID_VALUE, "cigemm_linear_f32: bad activation %d", (int)act);
  cigemmStatus_t st = check_gemm_args(h, "cigemm_linear_f32", M, N, K, X, ldx, W, ldw, N, out, ldo);
  if (st != CIGEMM_STATUS_SUCCESS || M == 0 || N == 0) return st;
  BiasAct ba{bias, act == CIGEMM_ACT_RELU};
  if (!dispatch_f32(h, M, N, K, X, ldx, W, ldw, out, ldo, &ba))
    return algo_refused(h, "cigemm_linear_f32");
  return check_launch(h, "cigemm_linear_f32");
}

static cigemmStatus_t gemm16(cigemmHandle_t h, const char* name, bool bf16, int64_t M, int64_t N,
                             int64_t K, const uint16_t* A, int64_t lda, const uint16_t* B,
                             int64_t ldb, uint16_t* C, int64_t ldc) {
  if (!valid(h)) return CIGEMM_STATUS_NOT_INITIALIZED;
  cigemmStatus_t st = check_gemm_args(h, name, M, N, K, A, lda, B, ldb, N, C, ldc);
  if (st != CIGEMM_STATUS_SUCCESS || M == 0 || N == 0) return st;
  bool ok = true;
  switch (h->algo) {
    case CIGEMM_ALGO_SKINNY: ok = launch_skinny_16(h, bf16, M, N, K, A, lda, B, ldb, C, ldc); break;
    case CIGEMM_ALGO_TILE: ok = launch_16b_mfma(h, bf16, M, N, K, A, lda, B, ldb, C, ldc); break;
    case CIGEMM_ALGO_SMALL: ok = false; break;
    case CIGEMM_ALGO_MFMA_ANY: ok = launch_mfma_any_16(h, bf16, M, N, K, A, lda, B, ldb, C, ldc); break;
    case CIGEMM_ALGO_GENERIC: launch_generic_16(h, bf16, M, N, K, A, lda, B, ldb, C, ldc); break;
    default:
      // decode shapes (M <= 32) first: they are bandwidth problems with their own kernel; what
      // neither that nor the tile kernel takes (odd N, unaligned rows) stays on the matrix cores
      if (!launch_skinny_16(h, bf16, M, N, K, A, lda, B, ldb, C, ldc) &&
          !launch_16b_mfma(h, bf16, M, N, K, A, lda, B, ldb, C, ldc) &&
          !launch_mfma_any_16(h, bf16, M, N, K, A, lda, B, ldb, C, ldc))
        launch_generic_16(h, bf16, M, N, K, A, lda, B, ldb, C, ldc);
  }
  if (!ok) return algo_refused(h, name);
  return check_launch(h, name);
}

cigemmStatus_t cigemm_gemm_f16(cigemmHandle_t h, int64_t M, int64_t N, int64_t K,
                               const uint16_t* A, int64_t lda, const uint16_t* B, int64_t ldb,
                               uint16_t* C, int64_t ldc) {
  return gemm16(h, "cigemm_gemm_f16", false, M, N, K, A, lda, B, ldb, C, ldc);
}

cigemmStatus_t cigemm_gemm_bf16(cigemmHandle_t h, int64_t M, int64_t N, int64_t K,
                                const uint16_t* A, int64_t lda, const uint16_t* B, int64_t ldb,
                                uint16_t* C, int64_t ldc) {
  return gemm16(h, "cigemm_gemm_bf16", true, M, N, K, A, lda, B, ldb, C, ldc);
}

static cigemmStatus_t gemm_i8(cigemmHandle_t h, const char* name, int64_t M, int64_t N, int64_t K,
                              const int8_t* A, int64_t lda, const int8_t* B, int64_t ldb,
                              cigemmBLayout_t b_layout, int32_t* C, int64_t ldc,
                              const DequantArgs* dq) {
  const bool b_nk = b_layout == CIGEMM_B_NK;
  bool ok = true;
  switch (h->algo) {
    case CIGEMM_ALGO_SKINNY: ok = launch_skinny_i8(h, M, N, K, A, lda, B, ldb, b_nk, C, ldc, dq); break;
    case CIGEMM_ALGO_TILE: ok = launch_i8_mfma(h, M, N, K, A, lda, B, ldb, b_nk, C, ldc, dq); break;
    case CIGEMM_ALGO_SMALL: ok = false; break;
    case CIGEMM_ALGO_MFMA_ANY:
      ok = launch_mfma_any_i8(h, M, N, K, A, lda, B, ldb, b_nk, C, ldc, dq);
      break;
    case CIGEMM_ALGO_GENERIC: launch_generic_i8(h, M, N, K, A, lda, B, ldb, b_nk, C, ldc, dq); break;
    default:
      if (!launch_skinny_i8(h, M, N, K, A, lda, B, ldb, b_nk, C, ldc, dq) &&
          !launch_i8_mfma(h, M, N, K, A, lda, B, ldb, b_nk, C, ldc, dq) &&
          !launch_mfma_any_i8(h, M, N, K, A, lda, B, ldb, b_nk, C, ldc, dq))
        launch_generic_i8(h, M, N, K, A, lda, B, ldb, b_nk, C, ldc, dq);
  }
  if (!ok) return algo_refused(h, name);
  return check_launch(h, name);
}

cigemmStatus_t cigemm_gemm_i8_i32(cigemmHandle_t h, int64_t M, int64_t N, int64_t K,
                                  const int8_t* A, int64_t lda, const int8_t* B, int64_t ldb,
                                  cigemmBLayout_t b_layout, int32_t* C, int64_t ldc) {
  if (!valid(h)) return CIGEMM_STATUS_NOT_INITIALIZED;
  if (b_layout != CIGEMM_B_KN && b_layout != CIGEMM_B_NK)
    return fail(h, CIGEMM_STATUS_INVALID_VALUE, "cigemm_gemm_i8_i32: bad b_layout %d",
                (int)b_layout);
  cigemmStatus_t st = check_gemm_args(h, "cigemm_gemm_i8_i32", M, N, K, A, lda, B, ldb,
                                      b_layout == CIGEMM_B_NK ? K : N, C, ldc);
  if (st != CIGEMM_STATUS_SUCCESS || M == 0 || N == 0) return st;
  return gemm_i8(h, "cigemm_gemm_i8_i32", M, N, K, A, lda, B, ldb, b_layout, C, ldc, nullptr);
}

cigemmStatus_t cigemm_gemm_i8_dequant(cigemmHandle_t h, int64_t M, int64_t N, int64_t K,
                                      const int8_t* A, int64_t lda, const int8_t* B, int64_t ldb,
                                      cigemmBLayout_t b_layout, const float* scaleA,
                                      cigemmScaleMode_t scaleA_mode, const float* scaleB,
                                      cigemmScaleMode_t scaleB_mode, void* out,
                                      cigemmOutType_t out_type, int64_t ldo, int32_t* acc_out,
                                      int64_t ldacc) {
  const char* name = "cigemm_gemm_i8_dequant";
  if (!valid(h)) return CIGEMM_STATUS_NOT_INITIALIZED;
  if (b_layout != CIGEMM_B_KN && b_layout != CIGEMM_B_NK)
    return fail(h, CIGEMM_STATUS_INVALID_VALUE, "%s: bad b_layout %d", name, (int)b_layout);
  if ((scaleA_mode != CIGEMM_SCALE_TENSOR && scaleA_mode != CIGEMM_SCALE_VECTOR) ||
      (scaleB_mode != CIGEMM_SCALE_TENSOR && scaleB_mode != CIGEMM_SCALE_VECTOR))
    return fail(h, CIGEMM_STATUS_INVALID_VALUE, "%s: bad scale mode", name);
  if (out_type != CIGEMM_OUT_F32 && out_type != CIGEMM_OUT_BF16)
    return fail(h, CIGEMM_STATUS_INVALID_VALUE, "%s: bad out_type %d", name, (int)out_type);
  cigemmStatus_t st = check_gemm_args(h, name, M, N, K, A, lda, B, ldb,
                                      b_layout == CIGEMM_B_NK ? K : N, out, ldo);
  if (st != CIGEMM_STATUS_SUCCESS || M == 0 || N == 0) return st;
  if (!scaleA || !scaleB) return fail(h, CIGEMM_STATUS_INVALID_VALUE, "%s: null scale pointer", name);
  if (acc_out && ldacc < N)
    return fail(h, CIGEMM_STATUS_INVALID_VALUE, "%s: ldacc=%lld < N=%lld", name, (long long)ldacc,
                (long long)N);
  DequantArgs dq{scaleA, scaleB, scaleA_mode == CIGEMM_SCALE_VECTOR,
                 scaleB_mode == CIGEMM_SCALE_VECTOR, out, out_type == CIGEMM_OUT_BF16, ldo,
                 acc_out, ldacc};
  return gemm_i8(h, name, M, N, K, A, lda, B, ldb, b_layout, nullptr, 0, &dq);
}

}  // extern "C"
