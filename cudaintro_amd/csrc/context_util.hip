// Helpers every kernel family shares, linked into the library and into the measurement
// library beside it: error recording on the context, the launch check, the composed kernel
// name of a tile-kernel call and the once-per-device dynamic-LDS attribute.
#include <cstdarg>

#include "common.h"

namespace cig {

cigemmStatus_t fail(cigemmContext* ctx, cigemmStatus_t st, const char* fmt, ...) {
  if (ctx) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(ctx->last_error, sizeof(ctx->last_error), fmt, ap);
    va_end(ap);
  }
  return st;
}

cigemmStatus_t check_launch(cigemmContext* ctx, const char* what) {
  if (ctx && ctx->pending_error[0]) {
    char msg[sizeof(ctx->pending_error)];
    memcpy(msg, ctx->pending_error, sizeof(msg));
    ctx->pending_error[0] = '\0';
    (void)hipGetLastError();
    return fail(ctx, CIGEMM_STATUS_INTERNAL_ERROR, "%s: %s", what, msg);
  }
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    if (ctx) ctx->ws_dirty = 1;  // see cigemmContext::ws_dirty
    return fail(ctx, CIGEMM_STATUS_EXECUTION_FAILED, "%s: HIP error: %s", what,
                hipGetErrorString(e));
  }
  return CIGEMM_STATUS_SUCCESS;
}

void set_tile_kernel_name(cigemmContext* ctx, const char* dtype, int k_elems, const char* suffix,
                          bool splitk) {
  char rows[24], waves[24];
  if (ctx->first_tile_rows) {
    snprintf(rows, sizeof(rows), "%d+%d", ctx->first_tile_rows, ctx->last_tile_rows);
    snprintf(waves, sizeof(waves), "w%d+w%d", ctx->first_waves, ctx->last_waves);
  } else {
    snprintf(rows, sizeof(rows), "%d", ctx->last_tile_rows);
    snprintf(waves, sizeof(waves), ctx->last_per_cu == 2 ? "w%dx2" : "w%d", ctx->last_waves);
  }
  snprintf(ctx->kernel_name, sizeof(ctx->kernel_name), "%s_mfma_%sx256x%d_%s_ring%d%s%s", dtype,
           rows, k_elems, waves, ctx->last_per_cu == 2 ? 3 : 4, suffix, splitk ? "_splitk" : "");
  ctx->last_kernel = ctx->kernel_name;
}

bool ensure_dynamic_lds(cigemmContext* ctx, const void* kernel, int bytes,
                        std::atomic<uint64_t>& done) {
  const uint64_t bit = 1ull << (ctx->device & 63);
  if (done.load(std::memory_order_acquire) & bit) return true;
  const hipError_t e =
      hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
  if (e != hipSuccess) {
    (void)hipGetLastError();
    snprintf(ctx->pending_error, sizeof(ctx->pending_error),
             "the device refused %d bytes of LDS per workgroup (%s)", bytes, hipGetErrorString(e));
    return false;
  }
  done.fetch_or(bit, std::memory_order_release);
  return true;
}

}  // namespace cig
