// Fused attention-score reduce feeding H2O / D2O.
//
// Stands in for CudaScoreReduceBackend::{reduce, reduce_per_layer}
// (crates/argus-extension-api/src/lib.rs:2938-2948); arithmetic of
// crates/techniques/attn-score/src/score_reduce.cu:13-62 and 64-91:
//   per token t: per layer  flat = sum_h p[l,h,t],  head[kv] = mean over the GQA group;
//   step = MAX over layers;  cumulative = cumulative * decay_factor + step.
// One thread per token, so consecutive lanes read consecutive floats of every score row.
#include "argus_hip_internal.hpp"

namespace {

constexpr int kMaxKvHeads = 16;

__global__ __launch_bounds__(256) void score_fused_reduce_kernel(
    const float *__restrict__ scores, float *__restrict__ importance,
    float *__restrict__ head_importance, float decay_factor, int n_layers, int n_heads_q,
    int n_kv_heads, int cache_seq_len, int64_t score_stride, int64_t max_seq_len) {
  const int t = blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= cache_seq_len) return;
  const int n_rep = n_heads_q / n_kv_heads;
  const float inv_rep = 1.0f / (float)n_rep;
  const int64_t layer_stride = (int64_t)n_heads_q * score_stride;

  float step_flat = 0.0f;
  float step_head[kMaxKvHeads];
#pragma unroll
  for (int kv = 0; kv < kMaxKvHeads; ++kv) step_head[kv] = 0.0f;

  for (int l = 0; l < n_layers; ++l) {
    const float *base = scores + l * layer_stride + t;
    float layer_flat = 0.0f;
#pragma unroll
    for (int kv = 0; kv < kMaxKvHeads; ++kv) {
      if (kv < n_kv_heads) {
        float g = 0.0f;
        for (int r = 0; r < n_rep; ++r) {
          const float w = base[(int64_t)(kv * n_rep + r) * score_stride];
          g += w;
          layer_flat += w;
        }
        step_head[kv] = fmaxf(step_head[kv], g * inv_rep);
      }
    }
    step_flat = fmaxf(step_flat, layer_flat);
  }

  importance[t] = importance[t] * decay_factor + step_flat;
#pragma unroll
  for (int kv = 0; kv < kMaxKvHeads; ++kv) {
    if (kv < n_kv_heads) {
      const int64_t i = (int64_t)kv * max_seq_len + t;
      head_importance[i] = head_importance[i] * decay_factor + step_head[kv];
    }
  }
}

__global__ __launch_bounds__(256) void score_reduce_per_layer_kernel(
    const float *__restrict__ scores, float *__restrict__ layer_flat, float decay_factor,
    int n_layers, int n_heads_q, int cache_seq_len, int64_t score_stride, int64_t max_seq_len) {
  const int t = blockIdx.x * blockDim.x + threadIdx.x;
  const int l = blockIdx.y;
  if (t >= cache_seq_len || l >= n_layers) return;
  const float *base = scores + (int64_t)l * n_heads_q * score_stride + t;
  float s = 0.0f;
  for (int h = 0; h < n_heads_q; ++h) s += base[(int64_t)h * score_stride];
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

ARGUS_API int argus_hip_score_reduce(argus_hip_ctx *ctx, const argus_hip_score_reduce_args *a) {
  int rc = check_args(ctx, a);
  if (rc != ARGUS_HIP_OK) return rc;
  if (!a->importance || !a->head_importance)
    return argus_fail(ctx, ARGUS_HIP_ERR_INVALID, "score_reduce: null cumulative buffer");
  // Same bound as the reference kernel's stack arrays (score_reduce.cu:11).
  if (a->n_kv_heads > (size_t)kMaxKvHeads)
    return argus_fail(ctx, ARGUS_HIP_ERR_UNSUPPORTED, "score_reduce: n_kv_heads %zu > 16", a->n_kv_heads);
  if (a->cache_seq_len == 0 || a->n_layers == 0) return ARGUS_HIP_OK;
  const int blocks = (int)((a->cache_seq_len + 255) / 256);
  hipLaunchKernelGGL(score_fused_reduce_kernel, dim3(blocks), dim3(256), 0, (hipStream_t)a->stream,
                     (const float *)a->score_buf, (float *)a->importance, (float *)a->head_importance,
                     a->decay_factor, (int)a->n_layers, (int)a->n_heads_q, (int)a->n_kv_heads,
                     (int)a->cache_seq_len, (int64_t)a->score_stride, (int64_t)a->max_seq_len);
  ARGUS_HIP_CHECK(ctx, hipGetLastError());
  return ARGUS_HIP_OK;
}

ARGUS_API int argus_hip_score_reduce_per_layer(argus_hip_ctx *ctx, const argus_hip_score_reduce_args *a) {
  int rc = check_args(ctx, a);
  if (rc != ARGUS_HIP_OK) return rc;
  if (!a->layer_flat_importance)
    return argus_fail(ctx, ARGUS_HIP_ERR_INVALID, "score_reduce_per_layer: null layer_flat_importance");
  if (a->cache_seq_len == 0 || a->n_layers == 0) return ARGUS_HIP_OK;
  if (a->n_layers > 65535) return argus_fail(ctx, ARGUS_HIP_ERR_UNSUPPORTED, "score_reduce_per_layer: n_layers");
  const int blocks = (int)((a->cache_seq_len + 255) / 256);
  hipLaunchKernelGGL(score_reduce_per_layer_kernel, dim3(blocks, (unsigned)a->n_layers), dim3(256), 0,
                     (hipStream_t)a->stream, (const float *)a->score_buf, (float *)a->layer_flat_importance,
                     a->decay_factor, (int)a->n_layers, (int)a->n_heads_q, (int)a->cache_seq_len,
                     (int64_t)a->score_stride, (int64_t)a->max_seq_len);
  ARGUS_HIP_CHECK(ctx, hipGetLastError());
  return ARGUS_HIP_OK;
}
