// Fused attention-score reduce feeding H2O / D2O.
//
// Stands in for CudaScoreReduceBackend::{reduce, reduce_per_layer}
// (crates/argus-extension-api/src/lib.rs:2938-2948); arithmetic of
// crates/techniques/attn-score/src/score_reduce.cu:13-62 and 64-91:
//   per token t: per layer  flat = sum_h p[l,h,t],  head[kv] = mean over the GQA group;
//   step = MAX over layers;  cumulative = cumulative * decay_factor + step.
// A lane owns one token, so consecutive lanes read consecutive floats of every score row; the
// layers of a 64-token tile are spread over the 16 waves of its workgroup (the maximum over layers
// is folded through LDS at the end), and a wave requests all rows of a GQA group before it adds them
// up: one thread per token with one load in flight, as in the reference kernel, ran at 0.5 TB/s on
// 32 layers x 32 heads x 32768 positions.
#include "argus_hip_internal.hpp"

#include <type_traits>

namespace {

// Probability of a logit given its row's (max, sum): the expression of the combine pass's rewrite, with
// the product rounded on its own (no fusing into the sums that follow), so that the reduce of a logits
// buffer equals the reduce of the probabilities bit for bit.
__device__ __forceinline__ float stat_weight_inv(float s, float m, float inv) {
  float p = __expf(s - m) * inv;
  asm("" : "+v"(p));  // the compiler sees a number, not a product it could fuse into the next addition
  return p;
}
__device__ __forceinline__ float stat_weight(float s, float m, float l) { return stat_weight_inv(s, m, 1.0f / l); }
// lane `src` (a constant) of x, through a scalar register
__device__ __forceinline__ float lane_value(float x, int src) {
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, x), src));
}

constexpr int kMaxKvHeads = 16;
constexpr int kReduceWaves = 16;

// NKV, NREP: KV heads and query heads per KV head when the pair is one of the common model shapes
// (the loop over heads is then straight-line code and all rows of a layer are requested together),
// 0, 0: any shape.
// STATS: the buffer holds logits and `stats` the (max, sum) of every (layer, head) row; a score is
// exp(s - max) * (1 / sum), the arithmetic of the rewrite the attention call left out.
template <int NKV, int NREP, bool STATS>
__global__ __launch_bounds__(64 * kReduceWaves) void score_fused_reduce_kernel(
    const float *__restrict__ scores, const float *__restrict__ stats, float *__restrict__ importance,
    float *__restrict__ head_importance, float decay_factor, int n_layers, int n_heads_q,
    int n_kv_heads, int cache_seq_len, int64_t score_stride, int64_t max_seq_len) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int t = blockIdx.x * 64 + lane;
  const int tc = min(t, cache_seq_len - 1);  // lanes past the end re-read the last token and store nothing
  const int n_rep = NREP > 0 ? NREP : n_heads_q / n_kv_heads;
  if constexpr (NKV > 0) n_kv_heads = NKV;
  const float inv_rep = 1.0f / (float)n_rep;
  const int64_t layer_stride = (int64_t)n_heads_q * score_stride;

  float step_flat = 0.0f;
  float step_head[kMaxKvHeads];
#pragma unroll
  for (int kv = 0; kv < kMaxKvHeads; ++kv) step_head[kv] = 0.0f;

  for (int l = wave; l < n_layers; l += kReduceWaves) {
    const float *base = scores + l * layer_stride + tc;
    const float *st = stats + (int64_t)l * n_heads_q * 2;  // uniform over the wave
    float layer_flat = 0.0f;
    if constexpr (NKV > 0) {
      float w[NKV * NREP];
#pragma unroll
      for (int h = 0; h < NKV * NREP; ++h) w[h] = __builtin_nontemporal_load(base + (int64_t)h * score_stride);
      if constexpr (STATS) {
        // lane h takes head h's reciprocal sum (one division per layer and wave, not one per score)
        static_assert(NKV * NREP <= 64, "one lane per head");
        const int hl = min(lane, NKV * NREP - 1);
        const float my_m = st[2 * hl], my_inv = 1.0f / st[2 * hl + 1];
#pragma unroll
        for (int h = 0; h < NKV * NREP; ++h) w[h] = stat_weight_inv(w[h], lane_value(my_m, h), lane_value(my_inv, h));
      }
#pragma unroll
      for (int kv = 0; kv < NKV; ++kv) {
        float g = 0.0f;
#pragma unroll
        for (int r = 0; r < NREP; ++r) {
          g += w[kv * NREP + r];
          layer_flat += w[kv * NREP + r];
        }
        step_head[kv] = fmaxf(step_head[kv], g * inv_rep);
      }
    } else {
#pragma unroll
      for (int kv = 0; kv < kMaxKvHeads; ++kv) {
        if (kv < n_kv_heads) {
          float g = 0.0f;
          for (int r = 0; r < n_rep; ++r) {
            float w = base[(int64_t)(kv * n_rep + r) * score_stride];
            if constexpr (STATS) w = stat_weight(w, st[2 * (kv * n_rep + r)], st[2 * (kv * n_rep + r) + 1]);
            g += w;
            layer_flat += w;
          }
          step_head[kv] = fmaxf(step_head[kv], g * inv_rep);
        }
      }
    }
    step_flat = fmaxf(step_flat, layer_flat);
  }

  // maximum over the waves: the upper half hands its values to the lower half, four times
  __shared__ float sh[kReduceWaves / 2][kMaxKvHeads + 1][64];
  for (int half = kReduceWaves / 2; half >= 1; half >>= 1) {
    if (wave >= half && wave < 2 * half) {
      sh[wave - half][0][lane] = step_flat;
#pragma unroll
      for (int kv = 0; kv < kMaxKvHeads; ++kv)
        if (kv < n_kv_heads) sh[wave - half][1 + kv][lane] = step_head[kv];
    }
    __syncthreads();
    if (wave < half) {
      step_flat = fmaxf(step_flat, sh[wave][0][lane]);
#pragma unroll
      for (int kv = 0; kv < kMaxKvHeads; ++kv)
        if (kv < n_kv_heads) step_head[kv] = fmaxf(step_head[kv], sh[wave][1 + kv][lane]);
    }
    __syncthreads();
  }
  if (wave != 0 || t >= cache_seq_len) return;

  importance[t] = importance[t] * decay_factor + step_flat;
#pragma unroll
  for (int kv = 0; kv < kMaxKvHeads; ++kv) {
    if (kv < n_kv_heads) {
      const int64_t i = (int64_t)kv * max_seq_len + t;
      head_importance[i] = head_importance[i] * decay_factor + step_head[kv];
    }
  }
}

template <bool STATS>
__global__ __launch_bounds__(256) void score_reduce_per_layer_kernel(
    const float *__restrict__ scores, const float *__restrict__ stats, float *__restrict__ layer_flat, float decay_factor,
    int n_layers, int n_heads_q, int cache_seq_len, int64_t score_stride, int64_t max_seq_len) {
  const int t = blockIdx.x * blockDim.x + threadIdx.x;
  const int l = blockIdx.y;
  // (max, 1 / sum) of the layer's heads, divided once per workgroup
  constexpr int kStatHeads = 256;
  __shared__ float sh_m[STATS ? kStatHeads : 1], sh_inv[STATS ? kStatHeads : 1];
  const float *st = stats + (int64_t)l * n_heads_q * 2;
  const bool shared_stats = STATS && n_heads_q <= kStatHeads;  // uniform
  if constexpr (STATS) {
    if (shared_stats) {
      if ((int)threadIdx.x < n_heads_q) {
        sh_m[threadIdx.x] = st[2 * threadIdx.x];
        sh_inv[threadIdx.x] = 1.0f / st[2 * threadIdx.x + 1];
      }
      __syncthreads();
    }
  }
  if (t >= cache_seq_len || l >= n_layers) return;
  const float *base = scores + (int64_t)l * n_heads_q * score_stride + t;
  auto weight = [&](float w, int h) {
    if constexpr (!STATS) return w;
    else return shared_stats ? stat_weight_inv(w, sh_m[h], sh_inv[h]) : stat_weight(w, st[2 * h], st[2 * h + 1]);
  };
  float s = 0.0f;
  int h = 0;
  for (; h + 8 <= n_heads_q; h += 8) {  // eight rows requested together, added in head order
    float w[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) w[i] = __builtin_nontemporal_load(base + (int64_t)(h + i) * score_stride);
#pragma unroll
    for (int i = 0; i < 8; ++i) s += weight(w[i], h + i);
  }
  for (; h < n_heads_q; ++h) s += weight(base[(int64_t)h * score_stride], h);
  const int64_t i = (int64_t)l * max_seq_len + t;
  layer_flat[i] = layer_flat[i] * decay_factor + s;
}

int check_args(argus_hip_ctx *ctx, const argus_hip_score_reduce_args *a) {
  if (!ctx || !a) return ARGUS_HIP_ERR_INVALID;
  if (!a->score_buf) return argus_fail(ctx, ARGUS_HIP_ERR_INVALID, "score_reduce: null score_buf");
  if (a->n_heads_q == 0 || a->n_kv_heads == 0 || a->n_heads_q % a->n_kv_heads)
    return argus_fail(ctx, ARGUS_HIP_ERR_INVALID, "score_reduce: heads %zu/%zu", a->n_heads_q, a->n_kv_heads);
  if (a->cache_seq_len > a->score_stride || a->cache_seq_len > a->max_seq_len)
    return argus_fail(ctx, ARGUS_HIP_ERR_INVALID, "score_reduce: cache_seq_len %zu exceeds stride %zu / max %zu",
                      a->cache_seq_len, a->score_stride, a->max_seq_len);
  return ARGUS_HIP_OK;
}

}  // namespace

ARGUS_API int argus_hip_score_reduce_ex(argus_hip_ctx *ctx, const argus_hip_score_reduce_args *a,
                                       const argus_hip_score_reduce_ext *ext) {
  int rc = check_args(ctx, a);
  if (rc != ARGUS_HIP_OK) return rc;
  if (!a->importance || !a->head_importance)
    return argus_fail(ctx, ARGUS_HIP_ERR_INVALID, "score_reduce: null cumulative buffer");
  // Same bound as the reference kernel's stack arrays (score_reduce.cu:11).
  if (a->n_kv_heads > (size_t)kMaxKvHeads)
    return argus_fail(ctx, ARGUS_HIP_ERR_UNSUPPORTED, "score_reduce: n_kv_heads %zu > 16", a->n_kv_heads);
  if (a->cache_seq_len == 0 || a->n_layers == 0) return ARGUS_HIP_OK;
  const float *stats = ext ? (const float *)ext->stats : nullptr;
  const dim3 grid((unsigned)((a->cache_seq_len + 63) / 64)), block(64 * kReduceWaves);
  auto launch = [&](auto kern) {
    hipLaunchKernelGGL(kern, grid, block, 0, (hipStream_t)a->stream, (const float *)a->score_buf, stats,
                       (float *)a->importance, (float *)a->head_importance, a->decay_factor, (int)a->n_layers,
                       (int)a->n_heads_q, (int)a->n_kv_heads, (int)a->cache_seq_len, (int64_t)a->score_stride,
                       (int64_t)a->max_seq_len);
  };
  auto pick = [&](auto nkv_c, auto nrep_c) {
    constexpr int NKV = decltype(nkv_c)::value, NREP = decltype(nrep_c)::value;
    if (stats) launch(score_fused_reduce_kernel<NKV, NREP, true>);
    else launch(score_fused_reduce_kernel<NKV, NREP, false>);
  };
  const int nkv = (int)a->n_kv_heads, nrep = (int)(a->n_heads_q / a->n_kv_heads);
  typedef std::integral_constant<int, 0> C0;
  typedef std::integral_constant<int, 2> C2;
  typedef std::integral_constant<int, 4> C4;
  typedef std::integral_constant<int, 6> C6;
  typedef std::integral_constant<int, 7> C7;
  typedef std::integral_constant<int, 8> C8;
  // (KV heads, group) of Llama-3 8B / 3.2 1B, Llama-3 70B, Qwen2.5 0.5B / 1.5B / 7B, Gemma-2 2B / 9B
  if (nkv == 8 && nrep == 4) pick(C8{}, C4{});
  else if (nkv == 8 && nrep == 8) pick(C8{}, C8{});
  else if (nkv == 2 && nrep == 7) pick(C2{}, C7{});
  else if (nkv == 2 && nrep == 6) pick(C2{}, C6{});
  else if (nkv == 4 && nrep == 7) pick(C4{}, C7{});
  else if (nkv == 4 && nrep == 2) pick(C4{}, C2{});
  else if (nkv == 8 && nrep == 2) pick(C8{}, C2{});
  else pick(C0{}, C0{});
  ARGUS_HIP_CHECK(ctx, hipGetLastError());
  return ARGUS_HIP_OK;
}

ARGUS_API int argus_hip_score_reduce(argus_hip_ctx *ctx, const argus_hip_score_reduce_args *a) {
  return argus_hip_score_reduce_ex(ctx, a, nullptr);
}

ARGUS_API int argus_hip_score_reduce_per_layer_ex(argus_hip_ctx *ctx, const argus_hip_score_reduce_args *a,
                                                 const argus_hip_score_reduce_ext *ext) {
  int rc = check_args(ctx, a);
  if (rc != ARGUS_HIP_OK) return rc;
  if (!a->layer_flat_importance)
    return argus_fail(ctx, ARGUS_HIP_ERR_INVALID, "score_reduce_per_layer: null layer_flat_importance");
  if (a->cache_seq_len == 0 || a->n_layers == 0) return ARGUS_HIP_OK;
  if (a->n_layers > 65535) return argus_fail(ctx, ARGUS_HIP_ERR_UNSUPPORTED, "score_reduce_per_layer: n_layers");
  const float *stats = ext ? (const float *)ext->stats : nullptr;
  const int blocks = (int)((a->cache_seq_len + 255) / 256);
  auto launch = [&](auto kern) {
    hipLaunchKernelGGL(kern, dim3(blocks, (unsigned)a->n_layers), dim3(256), 0, (hipStream_t)a->stream,
                       (const float *)a->score_buf, stats, (float *)a->layer_flat_importance, a->decay_factor,
                       (int)a->n_layers, (int)a->n_heads_q, (int)a->cache_seq_len, (int64_t)a->score_stride,
                       (int64_t)a->max_seq_len);
  };
  if (stats) launch(score_reduce_per_layer_kernel<true>);
  else launch(score_reduce_per_layer_kernel<false>);
  ARGUS_HIP_CHECK(ctx, hipGetLastError());
  return ARGUS_HIP_OK;
}

ARGUS_API int argus_hip_score_reduce_per_layer(argus_hip_ctx *ctx, const argus_hip_score_reduce_args *a) {
  return argus_hip_score_reduce_per_layer_ex(ctx, a, nullptr);
}
