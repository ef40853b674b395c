// Internal helpers shared by the gfx950 kernels and the C-ABI glue.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <vector>

#include "../../include/argus_hip.h"

#define ARGUS_API extern "C" __attribute__((visibility("default")))

// Environment switches, read once when the context is created.
struct ArgusEnv {
  bool decode_valu = false;    // ARGUS_HIP_DECODE=valu: vector-ALU decode kernel for A/B measurements
  bool scores_direct = false;  // ARGUS_HIP_SCORES=direct: score stores stay in the token loop
  bool kivi_valu = false;      // ARGUS_HIP_KIVI=valu: vector-ALU KIVI kernel
};

// What a launcher has learnt about one kernel on this context's device: resident workgroups per
// compute unit at the LDS size it launches with, and whether the dynamic-LDS limit was raised.
struct KernelFacts {
  const void *fn;
  uint32_t lds_bytes;
  int wgs_per_cu;
};

// First word of every argus_hip_ctx: entry points that receive a context through an untyped slot of
// the plugin interface check it before they touch anything else.
constexpr uint64_t kArgusCtxTag = 0x4152475553484950ull;  // "ARGUSHIP"

struct argus_hip_ctx {
  uint64_t tag = kArgusCtxTag;
  int device = 0;
  int compute_units = 0;
  hipDeviceProp_t props;
  ArgusEnv env;
  // Split-KV partial workspace: per (sequence, Q head, split) one (m, l) pair and one
  // un-normalised output row.  Sized at creation (argus_hip_create_ex) or by
  // argus_hip_reserve_workspace; a call that needs more grows it, which stalls the device.
  float *ws = nullptr;
  size_t ws_bytes = 0;
  // This device's copy of the library's static scratch array (looked up when the context is
  // created), and the lending of it: while ws_override is set, launchers take their partials from
  // there instead of `ws` and never allocate.
  float *scratch = nullptr;
  float *ws_override = nullptr;
  size_t ws_override_bytes = 0;
  // Scratch of the PFA side channel (logits of the trailing query rows); freed after a call that
  // made it large.
  float *pfa_ws = nullptr;
  size_t pfa_ws_bytes = 0;
  // Per-device launch facts (the kernels' function attributes are per device).
  std::vector<KernelFacts> facts;
  std::vector<const void *> lds_raised;
  // How the last split-KV decode call was cut (argus_hip_last_decode_plan).
  argus_hip_decode_plan plan = {};
  // Event triples of argus_hip_kernel_timing_begin/_end: before the dominant kernel, after it,
  // after the combine pass (or whatever else the call launched).
  std::vector<hipEvent_t> ev;
  size_t ev_used = 0;
  bool timing = false;
  bool timer_held = false;  // an enclosing KernelTimer brackets the launches: inner ones stay off
  char err[512] = {0};
};

// Brackets the launches issued during its lifetime when timing is armed: mark() closes the first
// interval (the dominant kernel), the destructor the second (the combine pass).
struct KernelTimer {
  argus_hip_ctx *ctx;
  hipStream_t stream;
  bool on, marked;
  KernelTimer(argus_hip_ctx *c, hipStream_t s) : ctx(c), stream(s), on(false), marked(false) {
    if (c->timing && !c->timer_held && c->ev_used + 3 <= c->ev.size()) {
      on = true;
      (void)hipEventRecord(c->ev[c->ev_used], s);
    }
  }
  void mark() {
    if (on && !marked) (void)hipEventRecord(ctx->ev[ctx->ev_used + 1], stream);
    marked = true;
  }
  ~KernelTimer() {
    if (on) {
      if (!marked) (void)hipEventRecord(ctx->ev[ctx->ev_used + 1], stream);
      (void)hipEventRecord(ctx->ev[ctx->ev_used + 2], stream);
      ctx->ev_used += 3;
    }
  }
};

inline int argus_fail(argus_hip_ctx *ctx, int code, const char *fmt, ...) {
  if (ctx) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(ctx->err, sizeof(ctx->err), fmt, ap);
    va_end(ap);
  }
  return code;
}

#define ARGUS_HIP_CHECK(ctx, expr)                                                          \
  do {                                                                                      \
    hipError_t e_ = (expr);                                                                 \
    if (e_ != hipSuccess)                                                                   \
      return argus_fail((ctx), ARGUS_HIP_ERR_RUNTIME, "%s: %s", #expr, hipGetErrorString(e_)); \
  } while (0)

// Ensures the context workspace holds at least `bytes`; reallocation frees the old buffer
// (hipFree synchronises the device, so no launch still reads it).  With a lent workspace
// (ws_override) nothing is allocated: a request beyond it fails with ARGUS_HIP_ERR_NOMEM.
int argus_ws_reserve(argus_hip_ctx *ctx, size_t bytes);
inline float *argus_ws(argus_hip_ctx *ctx) { return ctx->ws_override ? ctx->ws_override : ctx->ws; }

// Resident workgroups per compute unit of `fn` at `block` threads and `lds_bytes` of dynamic LDS,
// queried once per (kernel, LDS size) on this context.
template <typename F>
int argus_wgs_per_cu(argus_hip_ctx *ctx, F fn, int block, size_t lds_bytes) {
  for (const KernelFacts &k : ctx->facts)
    if (k.fn == (const void *)fn && k.lds_bytes == (uint32_t)lds_bytes) return k.wgs_per_cu;
  int n = 0;
  if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, fn, block, lds_bytes) != hipSuccess) {
    (void)hipGetLastError();
    n = 1;
  }
  n = n < 1 ? 1 : n;
  ctx->facts.push_back(KernelFacts{(const void *)fn, (uint32_t)lds_bytes, n});
  return n;
}
// Raises the dynamic-LDS limit of `fn` to `bytes`, once per kernel on this context.
template <typename F>
hipError_t argus_raise_lds_limit(argus_hip_ctx *ctx, F fn, int bytes) {
  for (const void *k : ctx->lds_raised)
    if (k == (const void *)fn) return hipSuccess;
  hipError_t e = hipFuncSetAttribute((const void *)fn, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
  if (e == hipSuccess) ctx->lds_raised.push_back((const void *)fn);
  return e;
}

#if defined(__HIPCC__)
// ---- wave64 cross-lane helpers ------------------------------------------------------------
// DPP moves stay inside a row of 16 lanes, which is all the 8/16-lane row groups need.
template <int CTRL>
__device__ __forceinline__ float dpp_mov(float x) {
  return __builtin_bit_cast(
      float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xf, 0xf, true));
}

// Lane i's value paired with that of lane i ^ 16 / i ^ 32 without an LDS round trip: the row swaps
// of this target exchange the odd 16-lane rows of one register with the even rows of another
// (v_permlane16_swap), or the wave's halves (v_permlane32_swap); started from two copies of x, the
// two results hold x of the lower and of the upper partner in every lane.
template <typename OP>
__device__ __forceinline__ float xor16_combine(float x, OP op) {
  const uint32_t b = __builtin_bit_cast(uint32_t, x);
  const auto sw = __builtin_amdgcn_permlane16_swap(b, b, false, false);
  return op(__builtin_bit_cast(float, (uint32_t)sw[0]), __builtin_bit_cast(float, (uint32_t)sw[1]));
}
template <typename OP>
__device__ __forceinline__ float xor32_combine(float x, OP op) {
  const uint32_t b = __builtin_bit_cast(uint32_t, x);
  const auto sw = __builtin_amdgcn_permlane32_swap(b, b, false, false);
  return op(__builtin_bit_cast(float, (uint32_t)sw[0]), __builtin_bit_cast(float, (uint32_t)sw[1]));
}
__device__ __forceinline__ float rows_allreduce_max(float x) {  // over lanes i, i^16, i^32, i^48
  const auto mx = [](float a, float b) { return fmaxf(a, b); };
  return xor32_combine(xor16_combine(x, mx), mx);
}

// All-reduce (sum) over aligned groups of LANES consecutive lanes; every lane gets the total.
template <int LANES>
__device__ __forceinline__ float group_allreduce_sum(float x) {
  if constexpr (LANES >= 2) x += dpp_mov<0xB1>(x);   // quad_perm [1,0,3,2]
  if constexpr (LANES >= 4) x += dpp_mov<0x4E>(x);   // quad_perm [2,3,0,1]
  if constexpr (LANES >= 8) x += dpp_mov<0x141>(x);  // row_half_mirror
  if constexpr (LANES >= 16) x += dpp_mov<0x140>(x); // row_mirror
  if constexpr (LANES >= 32) x += __shfl_xor(x, 16, 64);
  if constexpr (LANES >= 64) x += __shfl_xor(x, 32, 64);
  return x;
}

template <int LANES>
__device__ __forceinline__ float group_allreduce_max(float x) {
  if constexpr (LANES >= 2) x = fmaxf(x, dpp_mov<0xB1>(x));
  if constexpr (LANES >= 4) x = fmaxf(x, dpp_mov<0x4E>(x));
  if constexpr (LANES >= 8) x = fmaxf(x, dpp_mov<0x141>(x));
  if constexpr (LANES >= 16) x = fmaxf(x, dpp_mov<0x140>(x));
  if constexpr (LANES >= 32) x = fmaxf(x, __shfl_xor(x, 16, 64));
  if constexpr (LANES >= 64) x = fmaxf(x, __shfl_xor(x, 32, 64));
  return x;
}

__device__ __forceinline__ float wave_allreduce_sum(float x) { return group_allreduce_sum<64>(x); }
__device__ __forceinline__ float wave_allreduce_max(float x) { return group_allreduce_max<64>(x); }

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef float float4_t __attribute__((ext_vector_type(4)));

constexpr float kNegInf = -__builtin_huge_valf();

// Pins eight loaded values in registers at this point.  Without it the compiler sinks a load whose
// value is only used under a lane condition into a branch of its own, and a run of such loads
// becomes a chain of load-wait-load-wait round trips; pinned together, the eight loads are issued
// back to back and waited for once.
__device__ __forceinline__ void loaded8(float (&v)[8]) {
  asm volatile("" : "+v"(v[0]), "+v"(v[1]), "+v"(v[2]), "+v"(v[3]), "+v"(v[4]), "+v"(v[5]), "+v"(v[6]), "+v"(v[7]));
}

// x == hi + lo to ~2^-22 relative, both f16.  The value goes through an empty asm so the compiler
// sees one f32 number, not the expression that made it: otherwise it may round `hi` once straight
// from a fused product (fma_mix) for one use and twice (f32, then f16) for another, and at a
// rounding tie the two copies differ by an ulp, which makes `lo` belong to the wrong `hi`.
__device__ __forceinline__ void split_f16(float x, _Float16 &hi, _Float16 &lo) {
  asm("" : "+v"(x));
  hi = (_Float16)x;
  lo = (_Float16)(x - (float)hi);
}
#endif
