// Context, device query and the memory helpers behind the engine's Memory / Buffer impls.
#include "argus_hip_internal.hpp"

#include <cstring>
#include <new>

int argus_ws_reserve(argus_hip_ctx *ctx, size_t bytes) {
  if (bytes <= ctx->ws_bytes) return ARGUS_HIP_OK;
  size_t want = ctx->ws_bytes ? ctx->ws_bytes : (size_t)1 << 22;
  while (want < bytes) want <<= 1;
  float *p = nullptr;
  if (hipMalloc((void **)&p, want) != hipSuccess) {
    (void)hipGetLastError();
    return argus_fail(ctx, ARGUS_HIP_ERR_NOMEM, "workspace allocation of %zu bytes failed", want);
  }
  if (ctx->ws) (void)hipFree(ctx->ws);
  ctx->ws = p;
  ctx->ws_bytes = want;
  return ARGUS_HIP_OK;
}

ARGUS_API int argus_hip_abi_version(void) { return ARGUS_HIP_ABI_VERSION; }

ARGUS_API int argus_hip_create(int device, argus_hip_ctx **out) {
  if (!out) return ARGUS_HIP_ERR_INVALID;
  *out = nullptr;
  int n = 0;
  if (hipGetDeviceCount(&n) != hipSuccess || n <= 0) {
    (void)hipGetLastError();
    return ARGUS_HIP_ERR_RUNTIME;
  }
  if (device < 0 || device >= n) return ARGUS_HIP_ERR_INVALID;
  argus_hip_ctx *ctx = new (std::nothrow) argus_hip_ctx();
  if (!ctx) return ARGUS_HIP_ERR_NOMEM;
  ctx->device = device;
  if (hipSetDevice(device) != hipSuccess || hipGetDeviceProperties(&ctx->props, device) != hipSuccess) {
    (void)hipGetLastError();
    delete ctx;
    return ARGUS_HIP_ERR_RUNTIME;
  }
  ctx->compute_units = ctx->props.multiProcessorCount;
  int rc = argus_ws_reserve(ctx, (size_t)8 << 20);
  if (rc != ARGUS_HIP_OK) {
    delete ctx;
    return rc;
  }
  *out = ctx;
  return ARGUS_HIP_OK;
}

ARGUS_API int argus_hip_destroy(argus_hip_ctx *ctx) {
  if (!ctx) return ARGUS_HIP_ERR_INVALID;
  if (ctx->ws) (void)hipFree(ctx->ws);
  for (hipEvent_t e : ctx->ev) (void)hipEventDestroy(e);
  delete ctx;
  return ARGUS_HIP_OK;
}

ARGUS_API const char *argus_hip_last_error(const argus_hip_ctx *ctx) {
  return ctx ? ctx->err : "null context";
}

ARGUS_API int argus_hip_get_device_info(const argus_hip_ctx *ctx, argus_hip_device_info *info) {
  if (!ctx || !info) return ARGUS_HIP_ERR_INVALID;
  memset(info, 0, sizeof(*info));
  info->compute_units = ctx->props.multiProcessorCount;
  info->clock_mhz = ctx->props.clockRate / 1000;
  info->wavefront_size = ctx->props.warpSize;
  info->lds_bytes_per_block = (int32_t)ctx->props.sharedMemPerBlock;
  info->hbm_bytes = (int64_t)ctx->props.totalGlobalMem;
  strncpy(info->name, ctx->props.name, sizeof(info->name) - 1);
  strncpy(info->gcn_arch, ctx->props.gcnArchName, sizeof(info->gcn_arch) - 1);
  return ARGUS_HIP_OK;
}

ARGUS_API int argus_hip_malloc(argus_hip_ctx *ctx, size_t bytes, void **dev_ptr) {
  if (!ctx || !dev_ptr) return ARGUS_HIP_ERR_INVALID;
  *dev_ptr = nullptr;
  if (hipMalloc(dev_ptr, bytes ? bytes : 1) != hipSuccess) {
    (void)hipGetLastError();
    return argus_fail(ctx, ARGUS_HIP_ERR_NOMEM, "hipMalloc(%zu) failed", bytes);
  }
  return ARGUS_HIP_OK;
}

ARGUS_API int argus_hip_free(argus_hip_ctx *ctx, void *dev_ptr) {
  if (!ctx) return ARGUS_HIP_ERR_INVALID;
  if (dev_ptr) ARGUS_HIP_CHECK(ctx, hipFree(dev_ptr));
  return ARGUS_HIP_OK;
}

ARGUS_API int argus_hip_write_buffer(argus_hip_ctx *ctx, void *stream, void *dst_dev,
                                     const void *src_host, size_t bytes) {
  if (!ctx || (bytes && (!dst_dev || !src_host))) return ARGUS_HIP_ERR_INVALID;
  if (!bytes) return ARGUS_HIP_OK;
  ARGUS_HIP_CHECK(ctx, hipMemcpyAsync(dst_dev, src_host, bytes, hipMemcpyHostToDevice, (hipStream_t)stream));
  ARGUS_HIP_CHECK(ctx, hipStreamSynchronize((hipStream_t)stream));
  return ARGUS_HIP_OK;
}

ARGUS_API int argus_hip_read_buffer(argus_hip_ctx *ctx, void *stream, void *dst_host,
                                    const void *src_dev, size_t bytes) {
  if (!ctx || (bytes && (!dst_host || !src_dev))) return ARGUS_HIP_ERR_INVALID;
  if (!bytes) return ARGUS_HIP_OK;
  ARGUS_HIP_CHECK(ctx, hipMemcpyAsync(dst_host, src_dev, bytes, hipMemcpyDeviceToHost, (hipStream_t)stream));
  ARGUS_HIP_CHECK(ctx, hipStreamSynchronize((hipStream_t)stream));
  return ARGUS_HIP_OK;
}

ARGUS_API int argus_hip_copy_slice(argus_hip_ctx *ctx, void *stream, void *dst_dev,
                                   const void *src_dev, size_t bytes) {
  if (!ctx || (bytes && (!dst_dev || !src_dev))) return ARGUS_HIP_ERR_INVALID;
  if (!bytes) return ARGUS_HIP_OK;
  // hipMemcpyAsync handles overlapping device ranges as memmove does not; buffer_shift callers
  // (engine/src/backend.rs:1119) move towards lower addresses, which a forward copy handles,
  // but to stay safe for any overlap the shift goes through a non-overlapping check.
  const char *s = (const char *)src_dev;
  char *d = (char *)dst_dev;
  if ((d < s + bytes) && (s < d + bytes) && d != s)
    return argus_fail(ctx, ARGUS_HIP_ERR_UNSUPPORTED, "copy_slice: overlapping ranges");
  ARGUS_HIP_CHECK(ctx, hipMemcpyAsync(dst_dev, src_dev, bytes, hipMemcpyDeviceToDevice, (hipStream_t)stream));
  return ARGUS_HIP_OK;
}

ARGUS_API int argus_hip_synchronize(argus_hip_ctx *ctx, void *stream) {
  if (!ctx) return ARGUS_HIP_ERR_INVALID;
  ARGUS_HIP_CHECK(ctx, hipStreamSynchronize((hipStream_t)stream));
  return ARGUS_HIP_OK;
}

ARGUS_API int argus_hip_kernel_timing_begin(argus_hip_ctx *ctx, int32_t max_launches) {
  if (!ctx || max_launches <= 0) return ARGUS_HIP_ERR_INVALID;
  while (ctx->ev.size() < (size_t)max_launches * 2) {
    hipEvent_t e;
    ARGUS_HIP_CHECK(ctx, hipEventCreate(&e));
    ctx->ev.push_back(e);
  }
  ctx->ev_used = 0;
  ctx->timing = true;
  return ARGUS_HIP_OK;
}

ARGUS_API int argus_hip_kernel_timing_end(argus_hip_ctx *ctx, float *ms_out, int32_t capacity, int32_t *n_out) {
  if (!ctx || !n_out || (capacity > 0 && !ms_out)) return ARGUS_HIP_ERR_INVALID;
  ctx->timing = false;
  const size_t n = ctx->ev_used / 2;
  *n_out = (int32_t)n;
  if (n) ARGUS_HIP_CHECK(ctx, hipEventSynchronize(ctx->ev[ctx->ev_used - 1]));
  for (size_t i = 0; i < n && i < (size_t)capacity; ++i)
    ARGUS_HIP_CHECK(ctx, hipEventElapsedTime(&ms_out[i], ctx->ev[2 * i], ctx->ev[2 * i + 1]));
  ctx->ev_used = 0;
  return ARGUS_HIP_OK;
}
