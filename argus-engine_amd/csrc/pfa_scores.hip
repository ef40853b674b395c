// PFA side channel on the device: post-softmax probabilities of the trailing q_window query rows
// of a prefill chunk, summed over the rows and/or kept per row.
//
// Stands in for the host mirror prefill_attention_scores, engine/src/kv/standard_format.rs:1400-1510
// (which needs K read back from VRAM, standard_format.rs:1137-1173): same definition -- f32 dot in
// channel order, logit = dot * scale, row maximum, e = exp(logit - max), p = e / denom -- with the
// sums over rows and heads taken in the reference's order.  Two roundings differ: the dot uses a
// fused multiply-add per channel, and the denominator is a tree sum instead of a sum in key order.
//
// Kernels: the logits of every (head, row, key), once, into the workspace (pfa_logits_kernel: a lane
// keeps its key's row in registers, the query row is wave-uniform, so the channel-order chain is
// two vector instructions per element with no memory access inside); row statistics (max, denom)
// per (head, row); one thread per key walks the rows in order and adds into sum_out / writes the
// per-head rows; the head-mean layout walks heads then rows per (step, key).  When head_dim is not
// a multiple of 64, or the logits would not fit a 1 GiB workspace, the last three recompute each
// logit where they need it (the dot is deterministic), as the first version did: 13 ms instead of
// 0.1 ms for 32 heads x 32 rows x 8192 keys.
#include "argus_hip_internal.hpp"

namespace {

struct PfaParams {
  const float *q;
  const void *k;
  float *sum_out;
  float *per_row;
  float *stats;   // [n_heads_q, qwin, 2] = (max, denom)
  float *logits;  // [n_heads_q, qwin, prefix_len], or null: recompute
  int32_t n_heads_q, gqa, head_dim, seq_len, prefix_len;
  int64_t k_pos_stride, kv_head_stride;
  int32_t q_start_pos, qwin, qwin_start, window;  // window < 0: none
  int32_t per_head;
  int32_t exp_stored;  // the row-statistics pass has replaced every stored logit by exp(logit - row maximum)
  float scale, inv_heads;
};

__device__ __forceinline__ int row_lo(const PfaParams &p, int pos) {
  if (p.window < 0) return 0;
  const int w1 = p.window > 0 ? p.window - 1 : 0;
  return pos > w1 ? pos - w1 : 0;
}

// dot in channel order, one fused multiply-add per channel (the scalar reference loop rounds the
// product separately; the difference is some 1e-7 relative, far inside the 1e-4 bar on the scores)
template <typename K_T>
__device__ __forceinline__ float logit_of(const PfaParams &p, const float *qv, int h, int key) {
  const K_T *kv = (const K_T *)p.k + (int64_t)key * p.k_pos_stride + (int64_t)(h / p.gqa) * p.kv_head_stride;
  float dot = 0.0f;
  for (int d = 0; d < p.head_dim; ++d) dot = __builtin_fmaf(qv[d], (float)kv[d], dot);
  return __fmul_rn(dot, p.scale);
}

// The logit of (head h, window row `step`, key): stored, or recomputed.
template <typename K_T>
__device__ __forceinline__ float logit_at(const PfaParams &p, const float *qv, int h, int step, int key) {
  if (p.logits) return p.logits[((int64_t)h * p.qwin + step) * p.prefix_len + key];
  return logit_of<K_T>(p, qv, h, key);
}

// All logits of a 64-key tile of one KV head: lane = key, the (head of the group, window row) pairs
// are dealt to the four waves.  DC channels of the key's row sit in registers at a time (a longer
// row continues the chain from the partial dot kept in the workspace, which is the same chain); the
// query rows of up to 64 KB of pairs are staged in LDS and read back as broadcast 16-byte vectors,
// so the chain is one fused multiply-add per element with an LDS read every fourth.
template <typename K_T, int DC>
__global__ __launch_bounds__(256) void pfa_logits_kernel(const PfaParams p) {
  constexpr int PG = 16384 / DC;  // pairs per staged group
  __shared__ __attribute__((aligned(16))) float sq[16384];
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int key0 = blockIdx.x * 64, kvh = blockIdx.y;
  const int key = min(key0 + lane, p.prefix_len - 1);  // lanes past the end repeat the last key and store nothing
  const bool store = key0 + lane < p.prefix_len;
  const K_T *krow = (const K_T *)p.k + (int64_t)key * p.k_pos_stride + (int64_t)kvh * p.kv_head_stride;
  const int n_pairs = p.gqa * p.qwin;
  for (int c0 = 0; c0 < p.head_dim; c0 += DC) {
    float kreg[DC];
#pragma unroll
    for (int d = 0; d < DC; ++d) kreg[d] = (float)krow[c0 + d];
    for (int pg0 = 0; pg0 < n_pairs; pg0 += PG) {
      const int npg = min(PG, n_pairs - pg0);
      __syncthreads();  // the previous group's rows have been read
      for (int i = threadIdx.x; i < npg * (DC / 4); i += 256) {
        const int pi = pg0 + i / (DC / 4), c4 = i % (DC / 4);
        const int h = kvh * p.gqa + pi / p.qwin, r = p.qwin_start + pi % p.qwin;
        ((float4_t *)sq)[i] = *(const float4_t *)(p.q + ((int64_t)r * p.n_heads_q + h) * p.head_dim + c0 + 4 * c4);
      }
      __syncthreads();
      for (int pl = wave; pl < npg; pl += 4) {
        const int pi = pg0 + pl, g = pi / p.qwin, step = pi % p.qwin;  // wave-uniform
        const int h = kvh * p.gqa + g, pos = p.q_start_pos + p.qwin_start + step;
        if (key0 > pos || key0 + 63 < row_lo(p, pos)) continue;  // no key of the tile is visible to this row
        const float4_t *qv = (const float4_t *)(sq + pl * DC);
        float *slot = p.logits + ((int64_t)h * p.qwin + step) * p.prefix_len + key;
        float dot = c0 ? *slot : 0.0f;
#pragma unroll
        for (int d4 = 0; d4 < DC / 4; ++d4) {
          const float4_t qq = qv[d4];
#pragma unroll
          for (int e = 0; e < 4; ++e) dot = __builtin_fmaf(qq[e], kreg[4 * d4 + e], dot);
        }
        if (c0 + DC >= p.head_dim) dot = __fmul_rn(dot, p.scale);
        if (store) *slot = dot;
      }
    }
  }
}

// The same logits on the matrix cores: L[pair][key] = Q[pair] . K[key] as 32x32x16 f16 MFMAs, 32
// (head, window row) pairs of one KV head against 32 keys per tile.  The query rows are split into
// f16 hi + lo (an F32 key row too), so every product is exact and the dot keeps f32 accuracy; the
// summation order differs from the scalar chain at the 1e-7 level.  A = Q (lane: pair, registers: 8
// channels), B = K (lane: key): the accumulators come out with lane = key, register = pair, so a
// store instruction writes whole 128-byte runs of two score rows.
// A workgroup owns 32 KB of key rows of one KV head: its 256 threads fetch them with full-row
// coalesced loads into LDS (rows padded by 16 bytes), and after one barrier each of the four waves
// multiplies its own block of 32 pairs against every tile from there.  grid = (key chunks, KV heads,
// groups of 128 pairs).
typedef float float16_t __attribute__((ext_vector_type(16)));
template <typename K_T, int D>
__global__ __launch_bounds__(256) void pfa_logits_mfma_kernel(const PfaParams p) {
  constexpr int KK = D / 16;
  constexpr int kKeys = 32768 / (D * (int)sizeof(K_T)), kTiles = kKeys / 32;
  constexpr int kRowVecs = D * (int)sizeof(K_T) / 16, kRowBytes = D * (int)sizeof(K_T) + 16;
  constexpr int kVecsPerThread = kKeys * kRowVecs / 256;
  __shared__ __align__(16) unsigned char ks[kKeys * kRowBytes];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int ln = lane & 31, hl = lane >> 5;
  const int kvh = blockIdx.y, pb = (int)blockIdx.z * 4 + wave;
  const int n_pairs = p.gqa * p.qwin;
  const int pos_last = p.q_start_pos + p.seq_len - 1;  // no row sees a key beyond it
  const int chunk0 = (int)blockIdx.x * kKeys;
  if (chunk0 > pos_last) return;  // workgroup-uniform
  {
    float4_t v[kVecsPerThread];
#pragma unroll
    for (int j = 0; j < kVecsPerThread; ++j) {
      const int idx = (int)threadIdx.x + 256 * j;
      const int key = min(chunk0 + idx / kRowVecs, p.prefix_len - 1);
      v[j] = *(const float4_t *)((const char *)p.k + ((int64_t)key * p.k_pos_stride + (int64_t)kvh * p.kv_head_stride) * (int)sizeof(K_T) +
                                 16 * (idx % kRowVecs));
    }
#pragma unroll
    for (int j = 0; j < kVecsPerThread; ++j) {
      const int idx = (int)threadIdx.x + 256 * j;
      *(float4_t *)(ks + (idx / kRowVecs) * kRowBytes + 16 * (idx % kRowVecs)) = v[j];
    }
  }
  half8_t qh[KK], ql[KK];
  if (32 * pb < n_pairs) {
    const int pi = min(32 * pb + ln, n_pairs - 1);  // lanes past the last pair repeat it; their columns are not stored
    const int h = kvh * p.gqa + pi / p.qwin, r = p.qwin_start + pi % p.qwin;
    const float *qrow = p.q + ((int64_t)r * p.n_heads_q + h) * D + 8 * hl;
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
      const float4_t a = *(const float4_t *)(qrow + 16 * kk), b = *(const float4_t *)(qrow + 16 * kk + 4);
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        _Float16 hi, lo;
        split_f16(e < 4 ? a[e] : b[e - 4], hi, lo);
        qh[kk][e] = hi;
        ql[kk][e] = lo;
      }
    }
  }
  __syncthreads();
  if (32 * pb >= n_pairs) return;
  // score row of accumulator register i: pair 32 pb + 8 (i / 4) + 4 hl + i % 4
  int row_off[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int pm = 32 * pb + 8 * (i / 4) + 4 * hl + (i % 4);
    row_off[i] = pm < n_pairs ? ((kvh * p.gqa + pm / p.qwin) * p.qwin + pm % p.qwin) * p.prefix_len : -1;
  }
  for (int t = 0; t < kTiles; ++t) {
    const int key0 = chunk0 + 32 * t;
    if (key0 >= p.prefix_len || key0 > pos_last) break;  // wave-uniform
    const unsigned char *krow = ks + (32 * t + ln) * kRowBytes + 8 * hl * (int)sizeof(K_T);
    float16_t acc;
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = 0.0f;
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
      if constexpr (sizeof(K_T) == 2) {
        const half8_t kb = *(const half8_t *)(krow + 32 * kk);
        acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(qh[kk], kb, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(ql[kk], kb, acc, 0, 0, 0);
      } else {
        const float4_t a = *(const float4_t *)(krow + 64 * kk), b = *(const float4_t *)(krow + 64 * kk + 16);
        half8_t kbh, kbl;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          _Float16 hi, lo;
          split_f16(e < 4 ? a[e] : b[e - 4], hi, lo);
          kbh[e] = hi;
          kbl[e] = lo;
        }
        acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(qh[kk], kbh, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(ql[kk], kbh, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(qh[kk], kbl, acc, 0, 0, 0);
      }
    }
    if (key0 + ln < p.prefix_len) {
#pragma unroll
      for (int i = 0; i < 16; ++i)
        if (row_off[i] >= 0) __builtin_nontemporal_store(__fmul_rn(acc[i], p.scale), p.logits + (int64_t)row_off[i] + key0 + ln);
    }
  }
}

template <typename K_T>
__global__ __launch_bounds__(256) void pfa_rowstat_kernel(const PfaParams p) {
  __shared__ float red[4];
  const int step = blockIdx.x, h = blockIdx.y;
  const int r = p.qwin_start + step, pos = p.q_start_pos + r, lo = row_lo(p, pos);
  const float *qv = p.q + ((int64_t)r * p.n_heads_q + h) * p.head_dim;
  // With the logits stored, a thread keeps its first kHeld of them in registers: the loads go out
  // together and the second pass does not read them again. Longer rows continue through memory.
  constexpr int kHeld = 32;
  float held[kHeld];
  float *row = p.logits + ((int64_t)h * p.qwin + step) * p.prefix_len;
  const int tail = lo + (int)threadIdx.x + kHeld * 256;
  float m = kNegInf;
  if (p.exp_stored) {
#pragma unroll
    for (int i = 0; i < kHeld; ++i) {
      const int key = lo + (int)threadIdx.x + i * 256;
      held[i] = key <= pos ? row[key] : kNegInf;
    }
#pragma unroll
    for (int i = 0; i < kHeld; ++i) m = fmaxf(m, held[i]);
    for (int key = tail; key <= pos; key += 256) m = fmaxf(m, row[key]);
  } else {
    for (int key = lo + threadIdx.x; key <= pos; key += 256) m = fmaxf(m, logit_at<K_T>(p, qv, h, step, key));
  }
  m = wave_allreduce_max(m);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = m;
  __syncthreads();
  m = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
  __syncthreads();
  float s = 0.0f;
  if (p.exp_stored) {
    // the exponentials are what every later pass needs: they replace the logits in the workspace, so
    // no other kernel evaluates exp again
#pragma unroll
    for (int i = 0; i < kHeld; ++i) {
      const int key = lo + (int)threadIdx.x + i * 256;
      if (key <= pos) {
        const float e = expf(held[i] - m);
        row[key] = e;
        s += e;
      }
    }
    for (int key = tail; key <= pos; key += 256) {
      const float e = expf(row[key] - m);
      row[key] = e;
      s += e;
    }
  } else {
    for (int key = lo + threadIdx.x; key <= pos; key += 256) s += expf(logit_at<K_T>(p, qv, h, step, key) - m);
  }
  s = wave_allreduce_sum(s);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = s;
  __syncthreads();
  if (threadIdx.x == 0) {
    float *st = p.stats + ((int64_t)h * p.qwin + step) * 2;
    st[0] = m;
    st[1] = (red[0] + red[1]) + (red[2] + red[3]);
  }
}

// Probability of (head, window row, key): exp(logit - max) / denom, the exponential stored or recomputed.
template <typename K_T>
__device__ __forceinline__ float prob_at(const PfaParams &p, int h, int r, int step, int key) {
  const float *st = p.stats + ((int64_t)h * p.qwin + step) * 2;
  if (p.exp_stored) return __fdiv_rn(p.logits[((int64_t)h * p.qwin + step) * p.prefix_len + key], st[1]);
  const float *qv = p.q + ((int64_t)r * p.n_heads_q + h) * p.head_dim;
  return __fdiv_rn(expf(logit_at<K_T>(p, qv, h, step, key) - st[0]), st[1]);
}

// sum_out[h][key] += p over the rows in order; per-head per-row slots are written on the way.
// The stored exponentials are fetched kBatch rows at a time so the loads overlap; the additions keep
// their order.
constexpr int kBatch = 32;     // window rows fetched together by the sum pass (12.9 us; 8: 16.0 us)
constexpr int kHeadBatch = 8;  // heads fetched together by the head-mean pass, 1 MB apart (13.1 us; 32: 16.4 us)
template <typename K_T>
__global__ __launch_bounds__(256) void pfa_sum_kernel(const PfaParams p) {
  const int key = blockIdx.x * 256 + threadIdx.x, h = blockIdx.y;
  if (key >= p.prefix_len) return;
  float acc = p.sum_out ? p.sum_out[(int64_t)h * p.prefix_len + key] : 0.0f;
  if (p.exp_stored) {
    const float *base = p.logits + (int64_t)h * p.qwin * p.prefix_len + key;
    const float *st = p.stats + (int64_t)h * p.qwin * 2;
    for (int step0 = 0; step0 < p.qwin; step0 += kBatch) {
      float e[kBatch];
      bool live[kBatch];
#pragma unroll
      for (int j = 0; j < kBatch; ++j) {
        const int step = step0 + j, pos = p.q_start_pos + p.qwin_start + step;
        live[j] = step < p.qwin && key <= pos && key >= row_lo(p, pos);
        e[j] = live[j] ? base[(int64_t)step * p.prefix_len] : 0.0f;
      }
#pragma unroll
      for (int j = 0; j < kBatch; ++j) {
        if (!live[j]) continue;
        const int step = step0 + j;
        const float pr = __fdiv_rn(e[j], st[step * 2 + 1]);
        acc = __fadd_rn(acc, pr);
        if (p.per_row && p.per_head) p.per_row[((int64_t)step * p.n_heads_q + h) * p.prefix_len + key] = pr;
      }
    }
  } else {
    for (int step = 0; step < p.qwin; ++step) {
      const int r = p.qwin_start + step, pos = p.q_start_pos + r;
      if (key > pos || key < row_lo(p, pos)) continue;
      const float pr = prob_at<K_T>(p, h, r, step, key);
      acc = __fadd_rn(acc, pr);
      if (p.per_row && p.per_head) p.per_row[((int64_t)step * p.n_heads_q + h) * p.prefix_len + key] = pr;
    }
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
  if (p.exp_stored) {
    const float *base = p.logits + (int64_t)step * p.prefix_len + key;
    const float *st = p.stats + (int64_t)step * 2;
    for (int h0 = 0; h0 < p.n_heads_q; h0 += kHeadBatch) {
      float e[kHeadBatch];
#pragma unroll
      for (int j = 0; j < kHeadBatch; ++j) e[j] = h0 + j < p.n_heads_q ? base[(int64_t)(h0 + j) * p.qwin * p.prefix_len] : 0.0f;
#pragma unroll
      for (int j = 0; j < kHeadBatch; ++j)
        if (h0 + j < p.n_heads_q)
          acc = __fadd_rn(acc, __fmul_rn(__fdiv_rn(e[j], st[(int64_t)(h0 + j) * p.qwin * 2 + 1]), p.inv_heads));
    }
  } else {
    for (int h = 0; h < p.n_heads_q; ++h) acc = __fadd_rn(acc, __fmul_rn(prob_at<K_T>(p, h, r, step, key), p.inv_heads));
  }
  p.per_row[(int64_t)step * p.prefix_len + key] = acc;
}

template <typename K_T>
int launch(argus_hip_ctx *ctx, const PfaParams &p, hipStream_t stream) {
  if (p.logits) {
    // matrix cores when the rows allow 16-byte operand loads and the score rows 32-bit offsets
    const int kv_align = 16 / (int)sizeof(K_T);
    const bool mfma_ok = (p.head_dim == 64 || p.head_dim == 128 || p.head_dim == 256) && p.k_pos_stride % kv_align == 0 &&
                         p.kv_head_stride % kv_align == 0 && ((uintptr_t)p.k & 15) == 0 &&
                         (int64_t)p.n_heads_q * p.qwin * p.prefix_len < (1ll << 31);
    if (mfma_ok) {
      const int keys_per_wg = 32768 / (p.head_dim * (int)sizeof(K_T));
      const dim3 grid((unsigned)((p.prefix_len + keys_per_wg - 1) / keys_per_wg), (unsigned)(p.n_heads_q / p.gqa),
                      (unsigned)((p.gqa * p.qwin + 127) / 128));
      switch (p.head_dim) {
        case 64: hipLaunchKernelGGL((pfa_logits_mfma_kernel<K_T, 64>), grid, dim3(256), 0, stream, p); break;
        case 128: hipLaunchKernelGGL((pfa_logits_mfma_kernel<K_T, 128>), grid, dim3(256), 0, stream, p); break;
        default: hipLaunchKernelGGL((pfa_logits_mfma_kernel<K_T, 256>), grid, dim3(256), 0, stream, p); break;
      }
    } else {
      const dim3 grid((unsigned)((p.prefix_len + 63) / 64), (unsigned)(p.n_heads_q / p.gqa));
      if (p.head_dim % 128 == 0) hipLaunchKernelGGL((pfa_logits_kernel<K_T, 128>), grid, dim3(256), 0, stream, p);
      else hipLaunchKernelGGL((pfa_logits_kernel<K_T, 64>), grid, dim3(256), 0, stream, p);
    }
    ARGUS_HIP_CHECK(ctx, hipGetLastError());
  }
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
  const size_t stat_bytes = ((size_t)p.n_heads_q * p.qwin * 2 * sizeof(float) + 255) / 256 * 256;
  const size_t logit_bytes = (size_t)p.n_heads_q * p.qwin * p.prefix_len * sizeof(float);
  const bool keep_logits = p.head_dim % 64 == 0 && logit_bytes <= ((size_t)1 << 30) && ((uintptr_t)a->q & 15) == 0;
  // The logits live in a scratch buffer of their own (not the split-KV workspace, which stays at the
  // size the decode calls need).  It is kept between calls while small; a call that made it larger
  // than kKeepBytes gives it back before returning, which costs one stream synchronisation per
  // prefill chunk and layer.
  constexpr size_t kKeepBytes = (size_t)64 << 20;
  const size_t need = stat_bytes + (keep_logits ? logit_bytes : 0);
  if (need > ctx->pfa_ws_bytes) {
    if (ctx->pfa_ws) {
      ARGUS_HIP_CHECK(ctx, hipFree(ctx->pfa_ws));  // synchronises: no earlier call still reads it
      ctx->pfa_ws = nullptr;
      ctx->pfa_ws_bytes = 0;
    }
    if (hipMalloc((void **)&ctx->pfa_ws, need) != hipSuccess) {
      (void)hipGetLastError();
      ctx->pfa_ws = nullptr;
      return argus_fail(ctx, ARGUS_HIP_ERR_NOMEM, "prefill_attention_scores: scratch of %zu bytes", need);
    }
    ctx->pfa_ws_bytes = need;
  }
  p.stats = ctx->pfa_ws;
  p.logits = keep_logits ? (float *)((char *)ctx->pfa_ws + stat_bytes) : nullptr;
  p.exp_stored = keep_logits ? 1 : 0;
  hipStream_t stream = (hipStream_t)a->stream;
  const int rc = a->k_dtype == ARGUS_HIP_F16 ? launch<_Float16>(ctx, p, stream) : launch<float>(ctx, p, stream);
  if (ctx->pfa_ws_bytes > kKeepBytes) {
    (void)hipStreamSynchronize(stream);
    (void)hipFree(ctx->pfa_ws);
    ctx->pfa_ws = nullptr;
    ctx->pfa_ws_bytes = 0;
  }
  return rc;
}
