// Pieces shared by the split-KV decode kernels (F16/F32 cache and KIVI-quantised cache):
// launch parameters, the soft-cap, the uniform-weights fallback and the split-combine pass.
#pragma once

#include "argus_hip_internal.hpp"

#include <algorithm>

namespace argus_decode {

struct DecodeParams {
  const float *q;
  const void *k;
  const void *v;
  float *out;
  float *scores;
  const int32_t *kv_index;
  float *ws_ml;  // [batch, Hq, nsplit, 2]
  float *ws_o;   // [batch, Hq, nsplit, D]
  int32_t n_heads_q, n_heads_kv, group;  // group = Hq / Hkv
  int32_t len, kv_start, chunk, nsplit;
  int32_t score_stride;
  int64_t row_stride;   // elements between consecutive token rows of one KV head
  int64_t head_stride;  // elements between KV heads
  int64_t q_bs, out_bs, kv_bs, score_bs, index_bs;
  float scale, softcap;
  int32_t direct;  // nsplit == 1 and no scores: first pass writes `out` itself
  int32_t slot_bound;  // slots an index list may name (the cache capacity)
  int32_t head_chunks; // vector-ALU kernel: workgroups per KV head (GQA groups wider than its head tile)
};

// cap * tanh(s / cap) with tanh(x) = 1 - 2 / (exp(2x) + 1); the argument is clamped where
// tanh is 1 to f32 precision so exp cannot overflow.  The caller handles NaN.
__device__ __forceinline__ float softcap_tanh(float s, float cap, float inv_cap) {
  float x = s * inv_cap;
  x = fminf(fmaxf(x, -15.0f), 15.0f);
  const float e = __expf(2.0f * x);
  return cap * (1.0f - 2.0f * __frcp_rn(e + 1.0f));
}

// Uniform-weights fallback of common.rs:561-577: out = mean of the attended V rows, every
// probability 1/len.  Only reached when no logit is finite, so speed is irrelevant.
template <typename KV_T>
__device__ void uniform_fallback(const DecodeParams &p, int b, int h, int D) {
  const int kvh = h / p.group;
  const KV_T *vb = (const KV_T *)p.v + (int64_t)b * p.kv_bs + (int64_t)kvh * p.head_stride;
  const int32_t *idx = p.kv_index ? p.kv_index + (int64_t)b * p.index_bs : nullptr;
  const float u = 1.0f / (float)p.len;
  for (int c = threadIdx.x; c < D; c += blockDim.x) {
    float acc = 0.0f;
    for (int t = 0; t < p.len; ++t) {
      const int64_t slot = idx ? idx[t] : (p.kv_start + t);
      acc += u * (float)vb[slot * p.row_stride + c];
    }
    p.out[(int64_t)b * p.out_bs + (int64_t)h * D + c] = acc;
  }
  if (p.scores) {
    float *srow = p.scores + (int64_t)b * p.score_bs + (int64_t)h * p.score_stride;
    for (int t = threadIdx.x; t < p.len; t += blockDim.x) srow[t] = u;
  }
}

// Fallback policies of the combine pass when a row has no finite logit.
template <typename KV_T>
struct UniformFallback {
  // Scalar reference behaviour (common.rs:561-577): uniform weights.
  static __device__ bool run(const DecodeParams &p, int b, int h, int D) {
    uniform_fallback<KV_T>(p, b, h, D);
    return true;
  }
};
struct NoFallback {
  // The reference KIVI kernels have no guard (kivi_attn.cu:252-390): NaN propagates.
  static __device__ bool run(const DecodeParams &, int, int, int) { return false; }
};

// Second pass: log-sum-exp merge of the splits of one (sequence, Q head); optional in-place
// logits -> probabilities rewrite of the score row.  The 256 threads are arranged as
// (split group) x (float4 column) so the loop over splits is short and the loads are wide.
constexpr int kMaxSplits = 128;

template <typename FALLBACK, int D>
__global__ __launch_bounds__(256) void decode_combine_kernel(const DecodeParams p) {
  constexpr int CQ = D / 4;                // float4 columns per row
  constexpr int NSG = 256 / CQ;            // split groups
  constexpr int PER = kMaxSplits / NSG;    // splits per thread at most
  const int h = blockIdx.x, b = blockIdx.y;
  const int64_t pbase = ((int64_t)b * p.n_heads_q + h) * p.nsplit;
  const int cq = threadIdx.x % CQ, sg = threadIdx.x / CQ;
  __shared__ float sh_w[kMaxSplits];
  __shared__ float sh_m, sh_l;
  __shared__ float4_t sh_o[NSG][CQ];
  // The pass is one memory round trip long if nothing waits on anything else, so the partial
  // outputs are requested before the (m, l) pairs that weight them.  Slots past the last split
  // re-read it and get weight zero.
  const int last = p.nsplit - 1;
  float4_t part[PER];
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    if (i * NSG > last) break;  // uniform
    part[i] = *(const float4_t *)(p.ws_o + (pbase + min(sg + i * NSG, last)) * D + 4 * cq);
  }
  if (threadIdx.x < 64) {
    constexpr int MLP = kMaxSplits / 64;
    float pm[MLP], pl[MLP];
#pragma unroll
    for (int i = 0; i < MLP; ++i) {
      const int s = min((int)threadIdx.x + 64 * i, last);
      pm[i] = p.ws_ml[(pbase + s) * 2];
      pl[i] = p.ws_ml[(pbase + s) * 2 + 1];
    }
    float mm = kNegInf;
#pragma unroll
    for (int i = 0; i < MLP; ++i) mm = fmaxf(mm, pm[i]);
    mm = wave_allreduce_max(mm);
    const float m_ref = (mm == kNegInf) ? 0.0f : mm;
    float ll = 0.0f;
#pragma unroll
    for (int i = 0; i < MLP; ++i) {
      const int s = threadIdx.x + 64 * i;
      const float w = (s <= last) ? __expf(pm[i] - m_ref) : 0.0f;
      sh_w[s] = w;
      ll += pl[i] * w;
    }
    ll = wave_allreduce_sum(ll);
    if (threadIdx.x == 0) {
      sh_m = mm;
      sh_l = ll;
    }
  }
  __syncthreads();
  const float mm = sh_m, ll = sh_l;
  if (!(ll > 0.0f && ll < __builtin_huge_valf())) {
    if (FALLBACK::run(p, b, h, D)) return;
  }
  const float inv = 1.0f / ll;  // non-finite when the fallback declined: NaN propagates
  float4_t o = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    if (i * NSG > last) break;
    o += part[i] * sh_w[sg + i * NSG];
  }
  sh_o[sg][cq] = o;
  __syncthreads();
  if (sg == 0) {
#pragma unroll
    for (int g = 1; g < NSG; ++g) o += sh_o[g][cq];
    *(float4_t *)(p.out + (int64_t)b * p.out_bs + (int64_t)h * D + 4 * cq) = o * inv;
  }
  if (p.scores) {
    float *srow = p.scores + (int64_t)b * p.score_bs + (int64_t)h * p.score_stride;
    for (int t = threadIdx.x; t < p.len; t += 256) srow[t] = __expf(srow[t] - mm) * inv;
  }
}

// Split count of the matrix-core kernels.  The grid is sized against the number of workgroups the
// device holds at once (`slots`): when the splits fill it in one round every workgroup starts
// together and streams an equal share, each wave requesting its next tile while it works on the
// current one; a partial extra round runs thinly occupied (one 32K-token sequence: 2 rounds of
// 2-tile waves were 10 % slower than 1 round of 4-tile waves).  Cost model, in units of one tile
// step with the device full: rounds x (tile steps per workgroup + 0.75 for set-up, merge and
// partial write-out).  Sets p.nsplit and p.chunk (a multiple of tile_rows).
inline void choose_splits(DecodeParams &p, int pairs, int tile_rows, int64_t slots) {
  const int max_splits = std::min((p.len + tile_rows - 1) / tile_rows, kMaxSplits);
  int nsplit = 1, chunk = (p.len + tile_rows - 1) / tile_rows * tile_rows;
  float best = 3.0e38f;
  for (int n = 1; n <= max_splits; ++n) {
    const int c = ((p.len + n - 1) / n + tile_rows - 1) / tile_rows * tile_rows;
    const int ns = (p.len + c - 1) / c;
    const int64_t rounds = ((int64_t)pairs * ns + slots - 1) / slots;
    const float cost = (float)rounds * ((float)(c / tile_rows) + 0.75f);
    if (cost < best) {
      best = cost;
      nsplit = ns;
      chunk = c;
    }
  }
  p.nsplit = nsplit;
  p.chunk = chunk;
}

// Matrix-core variant (decode_mfma.hip): F16 cache, contiguous slots, no soft-cap.
bool decode_mfma_supported(const DecodeParams &p, int D, int kv_dtype);
int launch_decode_mfma(argus_hip_ctx *ctx, DecodeParams &p, int D, int batch, hipStream_t stream);
// Block-quantised caches (decode_blocks.hip): ARGUS_HIP_Q4_0 / Q4_1 / Q8_0, dequantised in registers.
int launch_decode_blocks(argus_hip_ctx *ctx, DecodeParams &p, int D, int kv_dtype, int batch, hipStream_t stream);

}  // namespace argus_decode
