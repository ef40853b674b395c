// PFA side channel on the device: post-softmax probabilities of the trailing q_window query rows
// of a prefill chunk, summed over the rows and/or kept per row.
//
// Stands in for the host mirror prefill_attention_scores, engine/src/kv/standard_format.rs:1400-1510
// (which needs K read back from VRAM, standard_format.rs:1137-1173): same definition -- scalar f32
// dot in channel order (mul, then add), logit = dot * scale, row maximum, e = exp(logit - max),
// p = e / denom -- with the sums over rows and heads taken in the reference's order.  Only the
// denominator is summed in a different order (tree instead of key order).
//
// Three small kernels: row statistics (max, denom) per (head, row); then one thread per key walks
// the rows in order and adds into sum_out / writes the per-head rows; the head-mean layout walks
// heads then rows per (step, key).  The logits are recomputed instead of stored (the dot is
// deterministic), so the workspace is two floats per (head, row).
#include "argus_hip_internal.hpp"

namespace {

struct PfaParams {
  const float *q;
  const void *k;
  float *sum_out;
  float *per_row;
  float *stats;  // [n_heads_q, qwin, 2] = (max, denom)
  int32_t n_heads_q, gqa, head_dim, seq_len, prefix_len;
  int64_t k_pos_stride, kv_head_stride;
  int32_t q_start_pos, qwin, qwin_start, window;  // window < 0: none
  int32_t per_head;
  float scale, inv_heads;
};

__device__ __forceinline__ int row_lo(const PfaParams &p, int pos) {
  if (p.window < 0) return 0;
  const int w1 = p.window > 0 ? p.window - 1 : 0;
  return pos > w1 ? pos - w1 : 0;
}

// dot in channel order with separately rounded multiply and add, like the scalar reference loop
template <typename K_T>
__device__ __forceinline__ float logit_of(const PfaParams &p, const float *qv, int h, int key) {
  const K_T *kv = (const K_T *)p.k + (int64_t)key * p.k_pos_stride + (int64_t)(h / p.gqa) * p.kv_head_stride;
  float dot = 0.0f;
  for (int d = 0; d < p.head_dim; ++d) dot = __fadd_rn(dot, __fmul_rn(qv[d], (float)kv[d]));
  return __fmul_rn(dot, p.scale);
}

template <typename K_T>
__global__ __launch_bounds__(256) void pfa_rowstat_kernel(const PfaParams p) {
  __shared__ float red[4];
  const int step = blockIdx.x, h = blockIdx.y;
  const int r = p.qwin_start + step, pos = p.q_start_pos + r, lo = row_lo(p, pos);
  const float *qv = p.q + ((int64_t)r * p.n_heads_q + h) * p.head_dim;
  float m = kNegInf;
  for (int key = lo + threadIdx.x; key <= pos; key += 256) m = fmaxf(m, logit_of<K_T>(p, qv, h, key));
  m = wave_allreduce_max(m);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = m;
  __syncthreads();
  m = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
  __syncthreads();
  float s = 0.0f;
  for (int key = lo + threadIdx.x; key <= pos; key += 256) s += expf(logit_of<K_T>(p, qv, h, key) - m);
  s = wave_allreduce_sum(s);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = s;
  __syncthreads();
  if (threadIdx.x == 0) {
    float *st = p.stats + ((int64_t)h * p.qwin + step) * 2;
    st[0] = m;
    st[1] = (red[0] + red[1]) + (red[2] + red[3]);
  }
}

// sum_out[h][key] += p over the rows in order; per-head per-row slots are written on the way.
template <typename K_T>
__global__ __launch_bounds__(256) void pfa_sum_kernel(const PfaParams p) {
  const int key = blockIdx.x * 256 + threadIdx.x, h = blockIdx.y;
  if (key >= p.prefix_len) return;
  float acc = p.sum_out ? p.sum_out[(int64_t)h * p.prefix_len + key] : 0.0f;
  for (int step = 0; step < p.qwin; ++step) {
    const int r = p.qwin_start + step, pos = p.q_start_pos + r;
    if (key > pos || key < row_lo(p, pos)) continue;
    const float *st = p.stats + ((int64_t)h * p.qwin + step) * 2;
    const float *qv = p.q + ((int64_t)r * p.n_heads_q + h) * p.head_dim;
    const float pr = __fdiv_rn(expf(logit_of<K_T>(p, qv, h, key) - st[0]), st[1]);
    acc = __fadd_rn(acc, pr);
    if (p.per_row && p.per_head) p.per_row[((int64_t)step * p.n_heads_q + h) * p.prefix_len + key] = pr;
  }
  if (p.sum_out) p.sum_out[(int64_t)h * p.prefix_len + key] = acc;
}

// head-mean per-row layout: out[step][key] += p / n_heads_q over the heads in order
template <typename K_T>
__global__ __launch_bounds__(256) void pfa_headmean_kernel(const PfaParams p) {
  const int key = blockIdx.x * 256 + threadIdx.x, step = blockIdx.y;
  if (key >= p.prefix_len) return;
  const int r = p.qwin_start + step, pos = p.q_start_pos + r;
  if (key > pos || key < row_lo(p, pos)) return;
  float acc = p.per_row[(int64_t)step * p.prefix_len + key];
  for (int h = 0; h < p.n_heads_q; ++h) {
    const float *st = p.stats + ((int64_t)h * p.qwin + step) * 2;
    const float *qv = p.q + ((int64_t)r * p.n_heads_q + h) * p.head_dim;
    const float pr = __fdiv_rn(expf(logit_of<K_T>(p, qv, h, key) - st[0]), st[1]);
    acc = __fadd_rn(acc, __fmul_rn(pr, p.inv_heads));
  }
  p.per_row[(int64_t)step * p.prefix_len + key] = acc;
}

template <typename K_T>
int launch(argus_hip_ctx *ctx, const PfaParams &p, hipStream_t stream) {
  hipLaunchKernelGGL(pfa_rowstat_kernel<K_T>, dim3(p.qwin, p.n_heads_q), dim3(256), 0, stream, p);
  ARGUS_HIP_CHECK(ctx, hipGetLastError());
  const unsigned kb = (unsigned)((p.prefix_len + 255) / 256);
  if (p.sum_out || (p.per_row && p.per_head)) {
    hipLaunchKernelGGL(pfa_sum_kernel<K_T>, dim3(kb, p.n_heads_q), dim3(256), 0, stream, p);
    ARGUS_HIP_CHECK(ctx, hipGetLastError());
  }
  if (p.per_row && !p.per_head) {
    hipLaunchKernelGGL(pfa_headmean_kernel<K_T>, dim3(kb, p.qwin), dim3(256), 0, stream, p);
    ARGUS_HIP_CHECK(ctx, hipGetLastError());
  }
  return ARGUS_HIP_OK;
}

}  // namespace

ARGUS_API int argus_hip_prefill_attention_scores(argus_hip_ctx *ctx, const argus_hip_pfa_args *a) {
  if (!ctx || !a) return ARGUS_HIP_ERR_INVALID;
  if (!a->q || !a->k) return argus_fail(ctx, ARGUS_HIP_ERR_INVALID, "prefill_attention_scores: null tensor pointer");
  if (a->n_heads_q <= 0 || a->n_heads_kv <= 0 || a->n_heads_q % a->n_heads_kv || a->head_dim <= 0)
    return argus_fail(ctx, ARGUS_HIP_ERR_INVALID, "prefill_attention_scores: heads %d/%d head_dim %d", a->n_heads_q, a->n_heads_kv,
                      a->head_dim);
  if (a->seq_len <= 0 || a->q_start_pos < 0 || a->q_start_pos + a->seq_len > a->cache_seq_len || a->q_window < 0)
    return argus_fail(ctx, ARGUS_HIP_ERR_INVALID, "prefill_attention_scores: seq_len %d q_start_pos %d cache_seq_len %d", a->seq_len,
                      a->q_start_pos, a->cache_seq_len);
  if (a->k_dtype != ARGUS_HIP_F16 && a->k_dtype != ARGUS_HIP_F32)
    return argus_fail(ctx, ARGUS_HIP_ERR_UNSUPPORTED, "prefill_attention_scores: K dtype %d", a->k_dtype);
  if (!a->sum_out && !a->per_row_out) return ARGUS_HIP_OK;  // nothing armed
  PfaParams p{};
  p.q = (const float *)a->q;
  p.k = a->k;
  p.sum_out = (float *)a->sum_out;
  p.per_row = (float *)a->per_row_out;
  p.n_heads_q = a->n_heads_q;
  p.gqa = a->n_heads_q / a->n_heads_kv;
  p.head_dim = a->head_dim;
  p.seq_len = a->seq_len;
  p.prefix_len = a->cache_seq_len;
  p.k_pos_stride = a->k_pos_stride;
  p.kv_head_stride = a->kv_head_stride;
  p.q_start_pos = a->q_start_pos;
  p.qwin = a->q_window < a->seq_len ? a->q_window : a->seq_len;
  p.qwin_start = a->seq_len - p.qwin;
  p.window = a->has_window ? a->window : -1;
  p.per_head = a->per_row_per_head;
  p.scale = 1.0f / sqrtf((float)a->head_dim);
  p.inv_heads = 1.0f / (float)a->n_heads_q;
  if (p.qwin == 0) return ARGUS_HIP_OK;
  int rc = argus_ws_reserve(ctx, (size_t)p.n_heads_q * p.qwin * 2 * sizeof(float));
  if (rc != ARGUS_HIP_OK) return rc;
  p.stats = ctx->ws;
  hipStream_t stream = (hipStream_t)a->stream;
  return a->k_dtype == ARGUS_HIP_F16 ? launch<_Float16>(ctx, p, stream) : launch<float>(ctx, p, stream);
}
