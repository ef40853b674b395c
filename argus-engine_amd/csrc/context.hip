// Context, device query and the memory helpers behind the engine's Memory / Buffer impls.
#include "argus_hip_internal.hpp"

#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <new>

// Scratch of the entry point that allocates nothing (argus_hip_attention_gen_noalloc): the split-KV
// partials of one call.  Each device the library runs on holds its own copy of this array, at its
// own address, until the process ends.  Host code never uses the array's name as an address: the
// per-device address comes from hipGetSymbolAddress when a context is created on that device.
constexpr size_t kScratchBytes = (size_t)16 << 20;
static __device__ __align__(256) unsigned char scratch[kScratchBytes];
constexpr int kMaxDevices = 64;
static void *g_scratch_addr[kMaxDevices] = {nullptr};
static std::mutex g_scratch_lock;  // contexts may be created from several threads

// With `device` current: the address of that device's copy of `scratch`, looked up once per device.
static int scratch_lookup(argus_hip_ctx *ctx, int device) {
  if (device < 0 || device >= kMaxDevices) return ARGUS_HIP_OK;  // no scratch there: the entry point refuses
  std::lock_guard<std::mutex> hold(g_scratch_lock);
  if (!g_scratch_addr[device]) {
    void *ptr = nullptr;
    const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !ptr) {
      (void)hipGetLastError();
      return argus_fail(ctx, ARGUS_HIP_ERR_RUNTIME, "hipGetSymbolAddress(scratch): %s", hipGetErrorString(e));
    }
    g_scratch_addr[device] = ptr;
  }
  ctx->scratch = (float *)g_scratch_addr[device];
  return ARGUS_HIP_OK;
}

int argus_ws_reserve(argus_hip_ctx *ctx, size_t bytes) {
  if (ctx->ws_override) {
    if (bytes <= ctx->ws_override_bytes) return ARGUS_HIP_OK;
    return argus_fail(ctx, ARGUS_HIP_ERR_NOMEM,
                      "attention_gen_noalloc: the call needs %zu bytes of split-KV partials, the static scratch holds %zu "
                      "(use argus_hip_attention_gen, or fewer sequences per call)",
                      bytes, ctx->ws_override_bytes);
  }
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

namespace {
bool env_is(const char *name, const char *value) {
  const char *e = getenv(name);
  return e && strcmp(e, value) == 0;
}
}  // namespace

ARGUS_API int argus_hip_create_ex(int device, const argus_hip_create_opts *opts, argus_hip_ctx **out) {
  if (!out) return ARGUS_HIP_ERR_INVALID;
  *out = nullptr;
  if (opts && (opts->max_batch < 0 || opts->max_heads_q < 0 || opts->max_head_dim < 0)) return ARGUS_HIP_ERR_INVALID;
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
  ctx->env.decode_valu = env_is("ARGUS_HIP_DECODE", "valu");
  ctx->env.scores_direct = env_is("ARGUS_HIP_SCORES", "direct");
  ctx->env.kivi_valu = env_is("ARGUS_HIP_KIVI", "valu");
  // The split-KV partials of the largest call the caller announces: every (sequence, Q head) may be
  // cut into kMaxSplitsHint pieces of head_dim + 2 floats.  Without a hint 8 MiB, which covers 16
  // sequences of the Llama-3-8B head shape at the split counts the launchers choose.
  size_t want = (size_t)8 << 20;
  if (opts && opts->max_batch > 0 && opts->max_heads_q > 0 && opts->max_head_dim > 0) {
    const size_t n_part = (size_t)opts->max_batch * opts->max_heads_q * 128;
    want = std::max(want, n_part * ((size_t)opts->max_head_dim + 2) * sizeof(float) + 256);
  }
  int rc = argus_ws_reserve(ctx, want);
  if (rc == ARGUS_HIP_OK) rc = scratch_lookup(ctx, device);
  if (rc != ARGUS_HIP_OK) {
    if (ctx->ws) (void)hipFree(ctx->ws);
    delete ctx;
    return rc;
  }
  *out = ctx;
  return ARGUS_HIP_OK;
}

ARGUS_API int argus_hip_create(int device, argus_hip_ctx **out) { return argus_hip_create_ex(device, nullptr, out); }

ARGUS_API int argus_hip_reserve_workspace(argus_hip_ctx *ctx, size_t bytes) {
  if (!ctx) return ARGUS_HIP_ERR_INVALID;
  return argus_ws_reserve(ctx, bytes);
}

ARGUS_API int argus_hip_destroy(argus_hip_ctx *ctx) {
  if (!ctx) return ARGUS_HIP_ERR_INVALID;
  if (ctx->ws) (void)hipFree(ctx->ws);
  if (ctx->pfa_ws) (void)hipFree(ctx->pfa_ws);
  for (hipEvent_t e : ctx->ev) (void)hipEventDestroy(e);
  ctx->tag = 0;  // a stale pointer no longer passes for a context
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

// argus_hip_attention_gen with the split-KV partials in this device's copy of `scratch`: no
// hipMalloc, hipFree or other allocating call on the way.  The partials a launch reads are all
// written by the same launch's first pass, so nothing in the array has to start at zero.
ARGUS_API int argus_hip_attention_gen_noalloc(argus_hip_ctx *ctx, const argus_hip_attention_gen_args *args) {
  if (!ctx || !args) return ARGUS_HIP_ERR_INVALID;
  if (!ctx->scratch) return argus_fail(ctx, ARGUS_HIP_ERR_RUNTIME, "attention_gen_noalloc: no static scratch on device %d", ctx->device);
  ctx->ws_override = ctx->scratch;
  ctx->ws_override_bytes = kScratchBytes;
  const int rc = argus_hip_attention_gen(ctx, args);
  ctx->ws_override = nullptr;
  ctx->ws_override_bytes = 0;
  return rc;
}

ARGUS_API int argus_hip_last_decode_plan(const argus_hip_ctx *ctx, argus_hip_decode_plan *plan) {
  if (!ctx || !plan) return ARGUS_HIP_ERR_INVALID;
  *plan = ctx->plan;
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

ARGUS_API int argus_hip_write_buffer_range(argus_hip_ctx *ctx, void *stream, void *dst_dev, size_t dst_offset,
                                           const void *src_host, size_t bytes) {
  if (!ctx || (bytes && (!dst_dev || !src_host))) return ARGUS_HIP_ERR_INVALID;
  return argus_hip_write_buffer(ctx, stream, (char *)dst_dev + dst_offset, src_host, bytes);
}

ARGUS_API int argus_hip_copy_slice(argus_hip_ctx *ctx, void *stream, void *dst_dev,
                                   const void *src_dev, size_t bytes) {
  if (!ctx || (bytes && (!dst_dev || !src_dev))) return ARGUS_HIP_ERR_INVALID;
  if (!bytes || dst_dev == src_dev) return ARGUS_HIP_OK;
  // Backend::copy_slice copies between two tensors (engine/src/backend.rs:1119); ranges that
  // overlap inside one buffer belong to buffer_shift and are handed over to it.
  const char *s = (const char *)src_dev;
  char *d = (char *)dst_dev;
  if ((d < s + bytes) && (s < d + bytes)) return argus_hip_buffer_shift(ctx, stream, dst_dev, src_dev, bytes);
  ARGUS_HIP_CHECK(ctx, hipMemcpyAsync(dst_dev, src_dev, bytes, hipMemcpyDeviceToDevice, (hipStream_t)stream));
  return ARGUS_HIP_OK;
}

// Backend::buffer_shift is std::ptr::copy, i.e. memmove (engine/src/backend.rs:1085-1112): the
// ranges may overlap, as when a cache prefix is pruned or the KIVI residual ring moves its
// remaining rows to the front (engine/src/kv/quant_window_cache.rs:1820-1841).  The move is cut into
// pieces that are each a plain copy between disjoint ranges, issued in the order that never
// overwrites bytes still to be read (ascending addresses when the destination lies below the
// source, descending otherwise).  A piece is at most as long as the distance between the ranges;
// when that distance is short the pieces go through the workspace instead (source piece ->
// workspace -> destination piece), so the number of copies stays bytes / workspace size.
ARGUS_API int argus_hip_buffer_shift(argus_hip_ctx *ctx, void *stream, void *dst_dev, const void *src_dev, size_t bytes) {
  if (!ctx || (bytes && (!dst_dev || !src_dev))) return ARGUS_HIP_ERR_INVALID;
  if (!bytes || dst_dev == src_dev) return ARGUS_HIP_OK;
  const char *s = (const char *)src_dev;
  char *d = (char *)dst_dev;
  hipStream_t st = (hipStream_t)stream;
  if (!((d < s + bytes) && (s < d + bytes))) {
    ARGUS_HIP_CHECK(ctx, hipMemcpyAsync(dst_dev, src_dev, bytes, hipMemcpyDeviceToDevice, st));
    return ARGUS_HIP_OK;
  }
  const bool forward = d < s;
  const size_t dist = forward ? (size_t)(s - d) : (size_t)(d - s);
  constexpr size_t kDirectMin = (size_t)1 << 20;  // pieces shorter than this are staged instead
  const bool staged = dist < kDirectMin && dist < bytes && ctx->ws_bytes > dist;
  const size_t piece = staged ? ctx->ws_bytes : dist;
  const size_t n = (bytes + piece - 1) / piece;
  for (size_t i = 0; i < n; ++i) {
    const size_t k = forward ? i : n - 1 - i;
    const size_t off = k * piece, len = std::min(piece, bytes - off);
    if (staged) {
      ARGUS_HIP_CHECK(ctx, hipMemcpyAsync(ctx->ws, s + off, len, hipMemcpyDeviceToDevice, st));
      ARGUS_HIP_CHECK(ctx, hipMemcpyAsync(d + off, ctx->ws, len, hipMemcpyDeviceToDevice, st));
    } else {
      ARGUS_HIP_CHECK(ctx, hipMemcpyAsync(d + off, s + off, len, hipMemcpyDeviceToDevice, st));
    }
  }
  return ARGUS_HIP_OK;
}

ARGUS_API int argus_hip_synchronize(argus_hip_ctx *ctx, void *stream) {
  if (!ctx) return ARGUS_HIP_ERR_INVALID;
  ARGUS_HIP_CHECK(ctx, hipStreamSynchronize((hipStream_t)stream));
  return ARGUS_HIP_OK;
}

ARGUS_API int argus_hip_kernel_timing_begin(argus_hip_ctx *ctx, int32_t max_launches) {
  if (!ctx || max_launches <= 0) return ARGUS_HIP_ERR_INVALID;
  while (ctx->ev.size() < (size_t)max_launches * 3) {
    hipEvent_t e;
    ARGUS_HIP_CHECK(ctx, hipEventCreate(&e));
    ctx->ev.push_back(e);
  }
  ctx->ev_used = 0;
  ctx->timing = true;
  return ARGUS_HIP_OK;
}

ARGUS_API int argus_hip_kernel_timing_end2(argus_hip_ctx *ctx, float *ms_out, float *tail_ms_out, int32_t capacity,
                                           int32_t *n_out) {
  if (!ctx || !n_out || (capacity > 0 && !ms_out)) return ARGUS_HIP_ERR_INVALID;
  ctx->timing = false;
  const size_t n = ctx->ev_used / 3;
  *n_out = (int32_t)n;
  if (n) ARGUS_HIP_CHECK(ctx, hipEventSynchronize(ctx->ev[ctx->ev_used - 1]));
  for (size_t i = 0; i < n && i < (size_t)capacity; ++i) {
    ARGUS_HIP_CHECK(ctx, hipEventElapsedTime(&ms_out[i], ctx->ev[3 * i], ctx->ev[3 * i + 1]));
    if (tail_ms_out) ARGUS_HIP_CHECK(ctx, hipEventElapsedTime(&tail_ms_out[i], ctx->ev[3 * i + 1], ctx->ev[3 * i + 2]));
  }
  ctx->ev_used = 0;
  return ARGUS_HIP_OK;
}

ARGUS_API int argus_hip_kernel_timing_end(argus_hip_ctx *ctx, float *ms_out, int32_t capacity, int32_t *n_out) {
  return argus_hip_kernel_timing_end2(ctx, ms_out, nullptr, capacity, n_out);
}
