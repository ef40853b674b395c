/*
 * argus_oracle.c -- CPU restatement of the Argus reference attention hot path.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing the product ships may link, import or call
 * this file: it exists so tests/, __graft_entry__.smoke() and bench.py's
 * cpu_baseline leg have something to check the HIP path against (and to time
 * beside it).  Every function cites the reference source it follows; paths are
 * relative to the reference repository root.
 *
 * The reference is Rust and cannot be built in this environment, so this is a
 * restatement, pinned by the reference's own known-answer vectors and by
 * closed-form / f64-textbook checks in tests/test_oracle_*.py.
 *
 * Build: gcc -O3 -mavx2 -mfma -mf16c -fopenmp -shared -fPIC (see Makefile).
 */
#include <immintrin.h>
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ORACLE_API __attribute__((visibility("default")))

/* ------------------------------------------------------------------------- */
/* f16 <-> f32: `half` 2.7.1 `f16::from_f32` / `to_f32` are IEEE-754 RNE      */
/* conversions (Cargo.lock:941-942); F16C implements the same rounding.       */
/* ------------------------------------------------------------------------- */
static inline float h2f(uint16_t h) { return _cvtsh_ss(h); }
static inline uint16_t f2h(float f) {
  return _cvtss_sh(f, _MM_FROUND_TO_NEAREST_INT | _MM_FROUND_NO_EXC);
}

ORACLE_API void oracle_f32_to_f16(const float *src, uint16_t *dst, int64_t n) {
  for (int64_t i = 0; i < n; ++i) dst[i] = f2h(src[i]);
}
ORACLE_API void oracle_f16_to_f32(const uint16_t *src, float *dst, int64_t n) {
  for (int64_t i = 0; i < n; ++i) dst[i] = h2f(src[i]);
}

/* LCG used by the reference's unit tests
 * (engine/src/backend/cpu/x86.rs:1546-1554,
 *  engine/tests/test_attention_flash_decoding.rs:44-52). */
ORACLE_API void oracle_gen_data(float *dst, int64_t n, uint32_t seed) {
  uint32_t s = seed;
  for (int64_t i = 0; i < n; ++i) {
    s = s * 1103515245u + 12345u;
    dst[i] = (float)(int16_t)(s >> 16) / 32768.0f;
  }
}

/* KV element offset: layout rule of engine/src/backend/cpu/x86.rs:195-198,
 * 225-229 (HeadMajor (kv_h*capacity+t)*d, SeqMajor (t*Hkv+kv_h)*d). */
static inline int64_t kv_off(int head_major, int64_t kv_h, int64_t t,
                             int64_t capacity, int64_t n_kv, int64_t d) {
  return head_major ? (kv_h * capacity + t) * d : (t * n_kv + kv_h) * d;
}

/* ------------------------------------------------------------------------- */
/* a-1 scalar: CpuBackendCommon::attention_gen                                */
/*   engine/src/backend/cpu/common.rs:359-675 (F32 arm 395-470, F16 arm       */
/*   471-675), NaN / all -inf / bad-sum guards 555-584.                       */
/*   kv_dtype: 0 = F32, 1 = F16.                                              */
/*   Extensions that the reference CPU path does not have, used only to check */
/*   the HIP kernel's extra arguments:                                        */
/*     softcap > 0: s = cap*tanh(s/cap) after *scale, definition from         */
/*       engine/kernels/flash_attn_f32_f16.cl:563-565;                        */
/*     kv_index != NULL: logical token t lives in physical slot kv_index[t]   */
/*       (gather-then-attend of engine/src/kv/standard_format.rs:2052-2184).  */
/* ------------------------------------------------------------------------- */
ORACLE_API int oracle_attention_gen_scalar(
    const float *q, const void *k_cache, const void *v_cache, float *out,
    int num_heads_q, int num_heads_kv, int head_dim, int cache_seq_len,
    int capacity, int head_major, int kv_dtype, float *scores_out,
    int64_t scores_stride, float softcap, const int32_t *kv_index) {
  if (kv_dtype != 0 && kv_dtype != 1) return -1;
  if (num_heads_kv <= 0 || num_heads_q % num_heads_kv) return -1;
  const float scale = 1.0f / sqrtf((float)head_dim);
  const int gqa = num_heads_q / num_heads_kv;
#pragma omp parallel for schedule(static)
  for (int h = 0; h < num_heads_q; ++h) {
    const int kv_h = h / gqa;
    const float *qv = q + (int64_t)h * head_dim;
    float *scores = (float *)malloc(sizeof(float) * (size_t)(cache_seq_len > 0 ? cache_seq_len : 1));
    for (int t = 0; t < cache_seq_len; ++t) {
      const int64_t slot = kv_index ? kv_index[t] : t;
      const int64_t off = kv_off(head_major, kv_h, slot, capacity, num_heads_kv, head_dim);
      float s = 0.0f;
      if (kv_dtype == 0) {
        const float *kr = (const float *)k_cache + off;
        for (int d = 0; d < head_dim; ++d) s += qv[d] * kr[d];
      } else {
        const uint16_t *kr = (const uint16_t *)k_cache + off;
        for (int d = 0; d < head_dim; ++d) s += qv[d] * h2f(kr[d]);
      }
      s *= scale;
      if (softcap > 0.0f) s = softcap * tanhf(s / softcap);
      scores[t] = s;
    }
    /* NaN guard (common.rs:555-560). */
    for (int t = 0; t < cache_seq_len; ++t)
      if (isnan(scores[t])) scores[t] = -INFINITY;
    float max_v = -INFINITY;
    for (int t = 0; t < cache_seq_len; ++t) max_v = fmaxf(max_v, scores[t]);
    if (max_v == -INFINITY) {
      const float u = 1.0f / (float)cache_seq_len;
      for (int t = 0; t < cache_seq_len; ++t) scores[t] = u;
    } else {
      float sum_e = 0.0f;
      for (int t = 0; t < cache_seq_len; ++t) {
        scores[t] = expf(scores[t] - max_v);
        sum_e += scores[t];
      }
      if (isnan(sum_e) || sum_e <= 0.0f || isinf(sum_e)) {
        const float u = 1.0f / (float)cache_seq_len;
        for (int t = 0; t < cache_seq_len; ++t) scores[t] = u;
      } else {
        for (int t = 0; t < cache_seq_len; ++t) scores[t] /= sum_e;
      }
    }
    if (scores_out)
      memcpy(scores_out + (int64_t)h * scores_stride, scores, sizeof(float) * (size_t)cache_seq_len);
    float *oh = out + (int64_t)h * head_dim;
    for (int d = 0; d < head_dim; ++d) oh[d] = 0.0f;
    for (int t = 0; t < cache_seq_len; ++t) {
      const float w = scores[t];
      const int64_t slot = kv_index ? kv_index[t] : t;
      const int64_t off = kv_off(head_major, kv_h, slot, capacity, num_heads_kv, head_dim);
      if (kv_dtype == 0) {
        const float *vr = (const float *)v_cache + off;
        for (int d = 0; d < head_dim; ++d) oh[d] += w * vr[d];
      } else {
        const uint16_t *vr = (const uint16_t *)v_cache + off;
        for (int d = 0; d < head_dim; ++d) oh[d] += w * h2f(vr[d]);
      }
    }
    free(scores);
  }
  return 0;
}

/* ------------------------------------------------------------------------- */
/* a-1 AVX2: CpuBackendAVX2::attention_gen                                    */
/*   engine/src/backend/cpu/x86.rs:178-357; helpers vec_dot_f16_f32_avx2      */
/*   601-666, vec_mad_f16_avx2 668-724, vec_dot_f32 1140-1178, exp_ps         */
/*   1263-1318, softmax_row 1474-1530.  No NaN guards (matches the source).   */
/*   This is the timed CPU baseline.                                          */
/* ------------------------------------------------------------------------- */
static inline float hsum8(__m256 x) {
  __m128 hi = _mm256_extractf128_ps(x, 1);
  __m128 lo = _mm256_castps256_ps128(x);
  __m128 s = _mm_add_ps(hi, lo);
  s = _mm_add_ps(s, _mm_movehl_ps(s, s));
  s = _mm_add_ss(s, _mm_movehdup_ps(s));
  return _mm_cvtss_f32(s);
}
static inline float hmax8(__m256 x) {
  __m128 hi = _mm256_extractf128_ps(x, 1);
  __m128 lo = _mm256_castps256_ps128(x);
  __m128 m = _mm_max_ps(hi, lo);
  m = _mm_max_ps(m, _mm_movehl_ps(m, m));
  m = _mm_max_ss(m, _mm_movehdup_ps(m));
  return _mm_cvtss_f32(m);
}

/* x86.rs:608-666 */
static float vec_dot_f16_f32_avx2(int k, const float *a, const uint16_t *b) {
  __m256 acc0 = _mm256_setzero_ps(), acc1 = acc0, acc2 = acc0, acc3 = acc0;
  int i = 0;
  for (; i + 32 <= k; i += 32) {
    __m256 b0 = _mm256_cvtph_ps(_mm_loadu_si128((const __m128i *)(b + i)));
    __m256 b1 = _mm256_cvtph_ps(_mm_loadu_si128((const __m128i *)(b + i + 8)));
    __m256 b2 = _mm256_cvtph_ps(_mm_loadu_si128((const __m128i *)(b + i + 16)));
    __m256 b3 = _mm256_cvtph_ps(_mm_loadu_si128((const __m128i *)(b + i + 24)));
    acc0 = _mm256_fmadd_ps(_mm256_loadu_ps(a + i), b0, acc0);
    acc1 = _mm256_fmadd_ps(_mm256_loadu_ps(a + i + 8), b1, acc1);
    acc2 = _mm256_fmadd_ps(_mm256_loadu_ps(a + i + 16), b2, acc2);
    acc3 = _mm256_fmadd_ps(_mm256_loadu_ps(a + i + 24), b3, acc3);
  }
  for (; i + 8 <= k; i += 8) {
    __m256 b0 = _mm256_cvtph_ps(_mm_loadu_si128((const __m128i *)(b + i)));
    acc0 = _mm256_fmadd_ps(_mm256_loadu_ps(a + i), b0, acc0);
  }
  acc0 = _mm256_add_ps(acc0, acc1);
  acc2 = _mm256_add_ps(acc2, acc3);
  acc0 = _mm256_add_ps(acc0, acc2);
  float sum = hsum8(acc0);
  for (; i < k; ++i) sum += a[i] * h2f(b[i]);
  return sum;
}

/* x86.rs:676-724 */
static void vec_mad_f16_avx2(int k, float *out, const uint16_t *v, float weight) {
  const __m256 w = _mm256_set1_ps(weight);
  int i = 0;
  /* main loop: 32 elements per iteration, as x86.rs:682-705 */
  for (; i + 32 <= k; i += 32) {
    __m256 v0 = _mm256_cvtph_ps(_mm_loadu_si128((const __m128i *)(v + i)));
    __m256 v1 = _mm256_cvtph_ps(_mm_loadu_si128((const __m128i *)(v + i + 8)));
    __m256 v2 = _mm256_cvtph_ps(_mm_loadu_si128((const __m128i *)(v + i + 16)));
    __m256 v3 = _mm256_cvtph_ps(_mm_loadu_si128((const __m128i *)(v + i + 24)));
    _mm256_storeu_ps(out + i, _mm256_fmadd_ps(w, v0, _mm256_loadu_ps(out + i)));
    _mm256_storeu_ps(out + i + 8, _mm256_fmadd_ps(w, v1, _mm256_loadu_ps(out + i + 8)));
    _mm256_storeu_ps(out + i + 16, _mm256_fmadd_ps(w, v2, _mm256_loadu_ps(out + i + 16)));
    _mm256_storeu_ps(out + i + 24, _mm256_fmadd_ps(w, v3, _mm256_loadu_ps(out + i + 24)));
  }
  for (; i + 8 <= k; i += 8) {
    __m256 v0 = _mm256_cvtph_ps(_mm_loadu_si128((const __m128i *)(v + i)));
    _mm256_storeu_ps(out + i, _mm256_fmadd_ps(w, v0, _mm256_loadu_ps(out + i)));
  }
  for (; i < k; ++i) out[i] += weight * h2f(v[i]);
}

/* x86.rs:1140-1178 */
static float vec_dot_f32_avx2(int n, const float *a, const float *b) {
  __m256 acc0 = _mm256_setzero_ps(), acc1 = acc0;
  int i = 0;
  for (; i + 16 <= n; i += 16) {
    acc0 = _mm256_fmadd_ps(_mm256_loadu_ps(a + i), _mm256_loadu_ps(b + i), acc0);
    acc1 = _mm256_fmadd_ps(_mm256_loadu_ps(a + i + 8), _mm256_loadu_ps(b + i + 8), acc1);
  }
  for (; i + 8 <= n; i += 8)
    acc0 = _mm256_fmadd_ps(_mm256_loadu_ps(a + i), _mm256_loadu_ps(b + i), acc0);
  acc0 = _mm256_add_ps(acc0, acc1);
  float sum = hsum8(acc0);
  for (; i < n; ++i) sum += a[i] * b[i];
  return sum;
}

static void vec_fma_f32_avx2(int n, float *out, const float *v, float weight) {
  const __m256 w = _mm256_set1_ps(weight);
  int i = 0;
  for (; i + 8 <= n; i += 8)
    _mm256_storeu_ps(out + i, _mm256_fmadd_ps(w, _mm256_loadu_ps(v + i), _mm256_loadu_ps(out + i)));
  for (; i < n; ++i) out[i] += weight * v[i];
}

/* x86.rs:1263-1318: Cephes-style polynomial exp, 8 lanes. */
static inline __m256 exp_ps(__m256 x) {
  const __m256 exp_hi = _mm256_set1_ps(88.37626f);
  const __m256 exp_lo = _mm256_set1_ps(-88.37626f);
  const __m256 log2ef = _mm256_set1_ps(1.44269504088896341f);
  const __m256 c1 = _mm256_set1_ps(0.6933594f);
  const __m256 c2 = _mm256_set1_ps(-2.1219444e-4f);
  const __m256 one = _mm256_set1_ps(1.0f);
  const __m256 p0 = _mm256_set1_ps(1.9875691e-4f);
  const __m256 p1 = _mm256_set1_ps(1.3982000e-3f);
  const __m256 p2 = _mm256_set1_ps(8.333452e-3f);
  const __m256 p3 = _mm256_set1_ps(4.166580e-2f);
  const __m256 p4 = _mm256_set1_ps(1.6666666e-1f);
  const __m256 p5 = _mm256_set1_ps(5.0000001e-1f);
  x = _mm256_min_ps(x, exp_hi);
  x = _mm256_max_ps(x, exp_lo);
  __m256 fx = _mm256_round_ps(_mm256_mul_ps(x, log2ef), _MM_FROUND_TO_NEAREST_INT | _MM_FROUND_NO_EXC);
  __m256 r = _mm256_fnmadd_ps(fx, c1, x);
  r = _mm256_fnmadd_ps(fx, c2, r);
  __m256 z = _mm256_mul_ps(r, r);
  __m256 y = p0;
  y = _mm256_fmadd_ps(y, r, p1);
  y = _mm256_fmadd_ps(y, r, p2);
  y = _mm256_fmadd_ps(y, r, p3);
  y = _mm256_fmadd_ps(y, r, p4);
  y = _mm256_fmadd_ps(y, r, p5);
  y = _mm256_fmadd_ps(y, z, r);
  y = _mm256_add_ps(y, one);
  __m256i n = _mm256_cvtps_epi32(fx);
  __m256 pow2n = _mm256_castsi256_ps(_mm256_slli_epi32(_mm256_add_epi32(n, _mm256_set1_epi32(0x7f)), 23));
  return _mm256_mul_ps(y, pow2n);
}

/* x86.rs:1474-1530 */
static void softmax_row_avx2(float *row, int dim) {
  __m256 max_v = _mm256_set1_ps(-INFINITY);
  int i = 0;
  for (; i + 8 <= dim; i += 8) max_v = _mm256_max_ps(max_v, _mm256_loadu_ps(row + i));
  float max_val = hmax8(max_v);
  for (; i < dim; ++i) max_val = fmaxf(max_val, row[i]);
  const __m256 mv = _mm256_set1_ps(max_val);
  __m256 sum_v = _mm256_setzero_ps();
  for (i = 0; i + 8 <= dim; i += 8) {
    __m256 e = exp_ps(_mm256_sub_ps(_mm256_loadu_ps(row + i), mv));
    _mm256_storeu_ps(row + i, e);
    sum_v = _mm256_add_ps(sum_v, e);
  }
  float sum_exp = hsum8(sum_v);
  for (; i < dim; ++i) {
    float e = expf(row[i] - max_val);
    row[i] = e;
    sum_exp += e;
  }
  const float inv = 1.0f / sum_exp;
  const __m256 inv_v = _mm256_set1_ps(inv);
  for (i = 0; i + 8 <= dim; i += 8) _mm256_storeu_ps(row + i, _mm256_mul_ps(_mm256_loadu_ps(row + i), inv_v));
  for (; i < dim; ++i) row[i] *= inv;
}

ORACLE_API int oracle_attention_gen_avx2(
    const float *q, const void *k_cache, const void *v_cache, float *out,
    int num_heads_q, int num_heads_kv, int head_dim, int cache_seq_len,
    int capacity, int head_major, int kv_dtype, float *scores_out,
    int64_t scores_stride, int n_threads) {
  if (kv_dtype != 0 && kv_dtype != 1) return -1;
  if (num_heads_kv <= 0 || num_heads_q % num_heads_kv) return -1;
  const float scale = 1.0f / sqrtf((float)head_dim);
  const int gqa = num_heads_q / num_heads_kv;
  if (n_threads <= 0) n_threads = num_heads_q;
  /* rayon par_chunks_mut(head_dim): one task per Q head (x86.rs:214-217). */
#pragma omp parallel for schedule(dynamic, 1) num_threads(n_threads)
  for (int h = 0; h < num_heads_q; ++h) {
    const int kv_h = h / gqa;
    const float *qv = q + (int64_t)h * head_dim;
    float *scores = (float *)malloc(sizeof(float) * (size_t)(cache_seq_len > 0 ? cache_seq_len : 1));
    for (int t = 0; t < cache_seq_len; ++t) {
      const int64_t off = kv_off(head_major, kv_h, t, capacity, num_heads_kv, head_dim);
      scores[t] = (kv_dtype == 0
                       ? vec_dot_f32_avx2(head_dim, qv, (const float *)k_cache + off)
                       : vec_dot_f16_f32_avx2(head_dim, qv, (const uint16_t *)k_cache + off)) *
                  scale;
    }
    softmax_row_avx2(scores, cache_seq_len);
    if (scores_out)
      memcpy(scores_out + (int64_t)h * scores_stride, scores, sizeof(float) * (size_t)cache_seq_len);
    float *oh = out + (int64_t)h * head_dim;
    for (int d = 0; d < head_dim; ++d) oh[d] = 0.0f;
    for (int t = 0; t < cache_seq_len; ++t) {
      const int64_t off = kv_off(head_major, kv_h, t, capacity, num_heads_kv, head_dim);
      if (kv_dtype == 0)
        vec_fma_f32_avx2(head_dim, oh, (const float *)v_cache + off, scores[t]);
      else
        vec_mad_f16_avx2(head_dim, oh, (const uint16_t *)v_cache + off, scores[t]);
    }
    free(scores);
  }
  return 0;
}

/* ------------------------------------------------------------------------- */
/* a-2 prefill: flash_attention_head / flash_attention_forward_strided        */
/*   engine/src/layers/attention.rs:78-221, 233-351 (scalar rayon path).      */
/*   window_size <= 0 means None.                                             */
/* ------------------------------------------------------------------------- */
static void flash_attention_head(const float *q, int64_t q_stride, const float *k,
                                 int64_t k_stride, const float *v, int64_t v_stride,
                                 float *out, int64_t out_stride, int q_len, int kv_len,
                                 int head_dim, int q_start_pos, int br, int bc,
                                 int window_size) {
  const float scale = 1.0f / sqrtf((float)head_dim);
  const int tr = (q_len + br - 1) / br;
  const int tc = (kv_len + bc - 1) / bc;
  float *oi = (float *)malloc(sizeof(float) * (size_t)br * head_dim);
  float *li = (float *)malloc(sizeof(float) * (size_t)br);
  float *mi = (float *)malloc(sizeof(float) * (size_t)br);
  float *sij = (float *)malloc(sizeof(float) * (size_t)bc);
  float *p_row = (float *)malloc(sizeof(float) * (size_t)bc);
  for (int i = 0; i < tr; ++i) {
    const int r_start = i * br;
    const int r_end = r_start + br < q_len ? r_start + br : q_len;
    const int cur_br = r_end - r_start;
    for (int x = 0; x < cur_br * head_dim; ++x) oi[x] = 0.0f;
    for (int r = 0; r < cur_br; ++r) { li[r] = 0.0f; mi[r] = -INFINITY; }
    for (int j = 0; j < tc; ++j) {
      const int c_start = j * bc;
      const int c_end = c_start + bc < kv_len ? c_start + bc : kv_len;
      const int cur_bc = c_end - c_start;
      const int64_t max_global_q = (int64_t)(r_end - 1) + q_start_pos;
      if (c_start > max_global_q) continue;
      if (window_size > 0) {
        const int64_t min_global_q = (int64_t)r_start + q_start_pos;
        if ((int64_t)c_end + window_size <= min_global_q + 1) continue;
      }
      for (int r = 0; r < cur_br; ++r) {
        const int global_r = r_start + r;
        float row_max = -INFINITY;
        int any_valid = 0;
        const int64_t global_q = (int64_t)global_r + q_start_pos;
        for (int c = 0; c < cur_bc; ++c) {
          sij[c] = -INFINITY;
          const int64_t global_c = c_start + c;
          const int causal_ok = global_c <= global_q;
          const int window_ok = window_size > 0 ? (global_c + window_size > global_q) : 1;
          if (causal_ok && window_ok) {
            float dot = 0.0f;
            const float *qp = q + (int64_t)global_r * q_stride;
            const float *kp = k + global_c * k_stride;
            for (int d = 0; d < head_dim; ++d) dot += qp[d] * kp[d];
            const float val = dot * scale;
            sij[c] = val;
            if (val > row_max) row_max = val;
            any_valid = 1;
          }
        }
        if (!any_valid) continue;
        const float m_prev = mi[r];
        const float m_new = fmaxf(m_prev, row_max);
        float l_new_part = 0.0f;
        for (int c = 0; c < cur_bc; ++c) {
          p_row[c] = 0.0f;
          if (sij[c] != -INFINITY) {
            p_row[c] = expf(sij[c] - m_new);
            l_new_part += p_row[c];
          }
        }
        const float alpha = (m_prev == -INFINITY) ? 0.0f : expf(m_prev - m_new);
        li[r] = li[r] * alpha + l_new_part;
        mi[r] = m_new;
        for (int d = 0; d < head_dim; ++d) {
          float pv_sum = 0.0f;
          for (int c = 0; c < cur_bc; ++c) {
            const int64_t global_c = c_start + c;
            const int causal_ok = global_c <= global_q;
            const int window_ok = window_size > 0 ? (global_c + window_size > global_q) : 1;
            if (causal_ok && window_ok) pv_sum += p_row[c] * v[global_c * v_stride + d];
          }
          oi[r * head_dim + d] = oi[r * head_dim + d] * alpha + pv_sum;
        }
      }
    }
    for (int r = 0; r < cur_br; ++r) {
      const int global_r = r_start + r;
      const float l_val = li[r];
      const float inv_l = (l_val == 0.0f) ? 0.0f : 1.0f / l_val;
      float *op = out + (int64_t)global_r * out_stride;
      for (int d = 0; d < head_dim; ++d) op[d] = oi[r * head_dim + d] * inv_l;
    }
  }
  free(oi); free(li); free(mi); free(sij); free(p_row);
}

ORACLE_API void oracle_flash_attention_forward_strided(
    const float *q, const float *k, const float *v, float *out, int n_heads_q,
    int n_heads_kv, int q_len, int kv_len, int head_dim, int64_t q_stride,
    int64_t k_stride, int64_t v_stride, int64_t out_stride, int64_t kv_head_stride,
    int q_start_pos, int br, int bc, int window_size, int n_threads) {
  const int n_rep = n_heads_q / n_heads_kv;
  if (n_threads <= 0) n_threads = n_heads_q;
  /* (0..n_heads_q).into_par_iter() (attention.rs:309). */
#pragma omp parallel for schedule(dynamic, 1) num_threads(n_threads)
  for (int h = 0; h < n_heads_q; ++h) {
    const int kv_h = h / n_rep;
    flash_attention_head(q + (int64_t)h * head_dim, q_stride, k + (int64_t)kv_h * kv_head_stride,
                         k_stride, v + (int64_t)kv_h * kv_head_stride, v_stride,
                         out + (int64_t)h * head_dim, out_stride, q_len, kv_len, head_dim,
                         q_start_pos, br, bc, window_size);
  }
}

/* StandardFormat::prefill_attention CPU arm, F16 / F32 HeadMajor KV:
 * engine/src/kv/standard_format.rs:1222-1252 (whole-cache F16->F32 dequant),
 * 1262-1310 (per-batch strides, q_start_pos = cache_seq_len - seq_len (:656),
 * Br = Bc = 32).  Q/out are [batch, seq_len, Hq, d] F32. */
ORACLE_API int oracle_prefill_attention(
    const float *q, const void *k_cache, const void *v_cache, float *out,
    int n_heads_q, int n_heads_kv, int seq_len, int cache_seq_len, int head_dim,
    int kv_capacity, int batch_size, int kv_dtype, int window_size, int n_threads) {
  if (kv_dtype != 0 && kv_dtype != 1) return -1;
  const int64_t kv_elems = (int64_t)batch_size * n_heads_kv * kv_capacity * head_dim;
  float *kf = NULL, *vf = NULL;
  const float *kp = (const float *)k_cache, *vp = (const float *)v_cache;
  if (kv_dtype == 1) {
    kf = (float *)malloc(sizeof(float) * (size_t)kv_elems);
    vf = (float *)malloc(sizeof(float) * (size_t)kv_elems);
    oracle_f16_to_f32((const uint16_t *)k_cache, kf, kv_elems);
    oracle_f16_to_f32((const uint16_t *)v_cache, vf, kv_elems);
    kp = kf; vp = vf;
  }
  const int64_t q_batch = (int64_t)seq_len * n_heads_q * head_dim;
  const int64_t kv_batch = (int64_t)kv_capacity * n_heads_kv * head_dim;
  for (int b = 0; b < batch_size; ++b) {
    oracle_flash_attention_forward_strided(
        q + b * q_batch, kp + b * kv_batch, vp + b * kv_batch, out + b * q_batch, n_heads_q,
        n_heads_kv, seq_len, cache_seq_len, head_dim, (int64_t)n_heads_q * head_dim, head_dim,
        head_dim, (int64_t)n_heads_q * head_dim, (int64_t)kv_capacity * head_dim,
        cache_seq_len - seq_len, 32, 32, window_size, n_threads);
  }
  free(kf); free(vf);
  return 0;
}

/* ------------------------------------------------------------------------- */
/* a-3 KIVI codec: crates/argus-kv-codec/src/lib.rs                           */
/*   BlockQ2_0 26-73 (12 B), BlockKVQ4 115-157 (20 B), BlockKVQ8 165-203      */
/*   (36 B).  Block = {d:f16, m:f16, qs[]}; codes use the f32 d.              */
/* ------------------------------------------------------------------------- */
static inline int kivi_block_bytes(int bits) { return 4 + 32 * bits / 8; }

/* Rust `f32::round` = half away from zero = roundf; `.clamp(0, hi) as u8`
 * saturates and maps NaN to 0. */
static inline uint8_t kivi_code(float x, float min_val, float id, float hi) {
  float r = roundf((x - min_val) * id);
  if (isnan(r)) return 0;
  if (r < 0.0f) r = 0.0f;
  if (r > hi) r = hi;
  return (uint8_t)r;
}

ORACLE_API int oracle_kivi_quantize_block(const float *src, int bits, uint8_t *dst) {
  if (bits != 2 && bits != 4 && bits != 8) return -1;
  /* Rust f32::min / f32::max ignore a NaN operand, like fminf / fmaxf. */
  float min_val = INFINITY, max_val = -INFINITY;
  for (int i = 0; i < 32; ++i) { min_val = fminf(min_val, src[i]); max_val = fmaxf(max_val, src[i]); }
  const float hi = (float)((1 << bits) - 1);
  const float range = max_val - min_val;
  const float d = range / hi;
  const float id = (d == 0.0f) ? 0.0f : 1.0f / d;
  const uint16_t dh = f2h(d), mh = f2h(min_val);
  memcpy(dst, &dh, 2);
  memcpy(dst + 2, &mh, 2);
  uint8_t *qs = dst + 4;
  if (bits == 2) {
    for (int i = 0; i < 8; ++i) {
      uint8_t byte = 0;
      for (int j = 0; j < 4; ++j) byte |= (uint8_t)(kivi_code(src[i * 4 + j], min_val, id, hi) << (j * 2));
      qs[i] = byte;
    }
  } else if (bits == 4) {
    for (int i = 0; i < 16; ++i) {
      const uint8_t lo = kivi_code(src[i * 2], min_val, id, hi);
      const uint8_t hi4 = kivi_code(src[i * 2 + 1], min_val, id, hi);
      qs[i] = (uint8_t)(lo | (hi4 << 4));
    }
  } else {
    for (int i = 0; i < 32; ++i) qs[i] = kivi_code(src[i], min_val, id, hi);
  }
  return 0;
}

ORACLE_API int oracle_kivi_dequantize_block(const uint8_t *blk, int bits, float *out) {
  if (bits != 2 && bits != 4 && bits != 8) return -1;
  uint16_t dh, mh;
  memcpy(&dh, blk, 2);
  memcpy(&mh, blk + 2, 2);
  const float d = h2f(dh), m = h2f(mh);
  const uint8_t *qs = blk + 4;
  for (int i = 0; i < 32; ++i) {
    uint8_t c;
    if (bits == 2) c = (qs[i / 4] >> ((i % 4) * 2)) & 0x03;
    else if (bits == 4) c = (qs[i / 2] >> ((i % 2) * 4)) & 0x0F;
    else c = qs[i];
    out[i] = (float)c * d + m;
  }
  return 0;
}

/* transition_bits between two quantised widths, quant_window_cache.rs:1350-1362 / 1421-1432:
 * dequantize_block then push_quantized per block, block order unchanged. */
ORACLE_API int oracle_kivi_requant(const uint8_t *src, uint8_t *dst, int64_t n_blocks, int old_bits, int new_bits) {
  if ((old_bits != 2 && old_bits != 4 && old_bits != 8) || (new_bits != 2 && new_bits != 4 && new_bits != 8)) return -1;
  const int ob = kivi_block_bytes(old_bits), nb = kivi_block_bytes(new_bits);
  float buf[32];
  for (int64_t i = 0; i < n_blocks; ++i) {
    oracle_kivi_dequantize_block(src + i * ob, old_bits, buf);
    oracle_kivi_quantize_block(buf, new_bits, dst + i * nb);
  }
  return 0;
}

/* ------------------------------------------------------------------------- */
/* a-3 KIVI container: QuantizedRecentWindowCache CPU path                    */
/*   update() engine/src/kv/quant_window_cache.rs:2518-2562 (lazy flush: when */
/*   the residual is full AND another token arrives), flush_residual()        */
/*   844-965 (K per channel: h -> group -> ch; V per token: h -> t -> block;  */
/*   then shift remainder).  Replays `n_tokens` single-token appends of       */
/*   SeqMajor [n_tokens, Hkv, d] F32 input.                                   */
/*   Outputs: qk/qv block bytes in push order (== the device order, see       */
/*   quant_window_cache.rs:1700-1722), residual [Hkv, res_cap, d] F32.        */
/* ------------------------------------------------------------------------- */
ORACLE_API int oracle_kivi_build(const float *k_in, const float *v_in, int n_tokens,
                                 int kv_heads, int head_dim, int res_cap, int bits,
                                 uint8_t *qk, uint8_t *qv, float *res_k, float *res_v,
                                 int *q_tokens_out, int *res_tokens_out) {
  if (res_cap <= 0 || res_cap % 32 || head_dim % 32) return -1;
  if (bits != 2 && bits != 4 && bits != 8) return -1;
  const int bb = kivi_block_bytes(bits);
  int64_t nk = 0, nv = 0;
  int q_tokens = 0, res_pos = 0;
  const int gs = 32;
  for (int s = 0; s < n_tokens; ++s) {
    if (res_pos >= res_cap) {
      const int n_groups = res_pos / gs;
      const int flush_tokens = n_groups * gs;
      for (int h = 0; h < kv_heads; ++h) {
        const int64_t head_base = (int64_t)h * res_cap * head_dim;
        for (int g = 0; g < n_groups; ++g) {
          const int tok_start = g * gs;
          for (int ch = 0; ch < head_dim; ++ch) {
            float vals[32];
            for (int t = 0; t < gs; ++t) vals[t] = res_k[head_base + (int64_t)(tok_start + t) * head_dim + ch];
            oracle_kivi_quantize_block(vals, bits, qk + nk * bb);
            ++nk;
          }
        }
      }
      const int bpt = head_dim / 32;
      for (int h = 0; h < kv_heads; ++h) {
        const int64_t head_base = (int64_t)h * res_cap * head_dim;
        for (int t = 0; t < flush_tokens; ++t)
          for (int b = 0; b < bpt; ++b) {
            oracle_kivi_quantize_block(res_v + head_base + (int64_t)t * head_dim + b * 32, bits, qv + nv * bb);
            ++nv;
          }
      }
      q_tokens += flush_tokens;
      const int remaining = res_pos - flush_tokens;
      if (remaining > 0)
        for (int h = 0; h < kv_heads; ++h) {
          const int64_t head_base = (int64_t)h * res_cap * head_dim;
          memmove(res_k + head_base, res_k + head_base + (int64_t)flush_tokens * head_dim, sizeof(float) * (size_t)remaining * head_dim);
          memmove(res_v + head_base, res_v + head_base + (int64_t)flush_tokens * head_dim, sizeof(float) * (size_t)remaining * head_dim);
        }
      res_pos = remaining;
    }
    for (int h = 0; h < kv_heads; ++h) {
      const int64_t src = ((int64_t)s * kv_heads + h) * head_dim;
      const int64_t dst = (int64_t)h * res_cap * head_dim + (int64_t)res_pos * head_dim;
      memcpy(res_k + dst, k_in + src, sizeof(float) * (size_t)head_dim);
      memcpy(res_v + dst, v_in + src, sizeof(float) * (size_t)head_dim);
    }
    ++res_pos;
  }
  *q_tokens_out = q_tokens;
  *res_tokens_out = res_pos;
  return 0;
}

/* assemble_view(): quant_window_cache.rs:1463-1553 -- dequantised SeqMajor
 * [total, Hkv, d] F32 view (quantised tokens first, then the residual). */
ORACLE_API int oracle_kivi_assemble_view(const uint8_t *qk, const uint8_t *qv,
                                         const float *res_k, const float *res_v,
                                         int q_tokens, int res_tokens, int kv_heads,
                                         int head_dim, int res_cap, int bits,
                                         float *attn_k, float *attn_v) {
  if (bits != 2 && bits != 4 && bits != 8) return -1;
  const int bb = kivi_block_bytes(bits);
  const int gs = 32, gpf = res_cap / gs, bpt = head_dim / 32;
  const int n_flush = q_tokens / res_cap;
  int64_t kb = 0, vb = 0;
  float buf[32];
  for (int f = 0; f < n_flush; ++f) {
    const int tok_base = f * res_cap;
    for (int h = 0; h < kv_heads; ++h)
      for (int g = 0; g < gpf; ++g)
        for (int ch = 0; ch < head_dim; ++ch) {
          oracle_kivi_dequantize_block(qk + kb * bb, bits, buf);
          ++kb;
          for (int t = 0; t < gs; ++t)
            attn_k[((int64_t)(tok_base + g * gs + t) * kv_heads + h) * head_dim + ch] = buf[t];
        }
    for (int h = 0; h < kv_heads; ++h)
      for (int t = 0; t < res_cap; ++t)
        for (int b = 0; b < bpt; ++b) {
          oracle_kivi_dequantize_block(qv + vb * bb, bits, buf);
          ++vb;
          memcpy(attn_v + ((int64_t)(tok_base + t) * kv_heads + h) * head_dim + b * 32, buf, sizeof(buf));
        }
  }
  for (int h = 0; h < kv_heads; ++h)
    for (int t = 0; t < res_tokens; ++t) {
      const int64_t o = ((int64_t)(q_tokens + t) * kv_heads + h) * head_dim;
      const int64_t r = (int64_t)h * res_cap * head_dim + (int64_t)t * head_dim;
      memcpy(attn_k + o, res_k + r, sizeof(float) * (size_t)head_dim);
      memcpy(attn_v + o, res_v + r, sizeof(float) * (size_t)head_dim);
    }
  return 0;
}

/* Fused KIVI attention, semantics of kernel_attn_gen_kivi_q{2,4,8}:
 *   crates/techniques/kivi/src/kivi_attn.cu:34-206 / 220-390 / 403-573
 *   (device block index math 71-77 / 256-262 K, 173-177 / 357-361 V; dequant
 *   code*d+m 213-218; residual [Hkv,res_cap,d] F32 270; score write 352-354).
 * Plain 3-pass softmax in f32, one Q head at a time. */
ORACLE_API int oracle_kivi_attention(const float *q, const uint8_t *qk, const uint8_t *qv,
                                     const float *res_k, const float *res_v, float *out,
                                     float *scores, int64_t score_stride, int num_heads_q,
                                     int num_heads_kv, int head_dim, int q_tokens,
                                     int res_tokens, int res_cap, float scale, int bits) {
  if (bits != 2 && bits != 4 && bits != 8) return -1;
  if (num_heads_q <= 0 || num_heads_kv <= 0) return -1;
  const int bb = kivi_block_bytes(bits);
  const int total = q_tokens + res_tokens;
  const int gpf = res_cap / 32, bpt = head_dim / 32;
  const int gqa = num_heads_q / num_heads_kv;
#pragma omp parallel for schedule(static)
  for (int h = 0; h < num_heads_q; ++h) {
    const int kv_head = h / gqa;
    const float *qp = q + (int64_t)h * head_dim;
    float *w = (float *)malloc(sizeof(float) * (size_t)(total > 0 ? total : 1));
    float buf[32];
    /* K: dequantise one channel block, scatter into 32 token scores. */
    for (int t = 0; t < total; ++t) w[t] = 0.0f;
    for (int g = 0; g < q_tokens / 32; ++g) {
      const int flush = g / gpf, gif = g % gpf;
      const int64_t block_idx = (int64_t)flush * num_heads_kv * gpf * head_dim +
                                (int64_t)kv_head * gpf * head_dim + (int64_t)gif * head_dim;
      for (int ch = 0; ch < head_dim; ++ch) {
        oracle_kivi_dequantize_block(qk + (block_idx + ch) * bb, bits, buf);
        for (int t = 0; t < 32; ++t) w[g * 32 + t] += qp[ch] * buf[t];
      }
    }
    for (int rt = 0; rt < res_tokens; ++rt) {
      const float *kp = res_k + (int64_t)kv_head * res_cap * head_dim + (int64_t)rt * head_dim;
      float s = 0.0f;
      for (int d = 0; d < head_dim; ++d) s += qp[d] * kp[d];
      w[q_tokens + rt] = s;
    }
    float mx = -INFINITY;
    for (int t = 0; t < total; ++t) { w[t] *= scale; mx = fmaxf(mx, w[t]); }
    float sum = 0.0f;
    for (int t = 0; t < total; ++t) { w[t] = expf(w[t] - mx); sum += w[t]; }
    for (int t = 0; t < total; ++t) w[t] /= sum;
    if (scores) memcpy(scores + (int64_t)h * score_stride, w, sizeof(float) * (size_t)total);
    float *oh = out + (int64_t)h * head_dim;
    for (int d = 0; d < head_dim; ++d) oh[d] = 0.0f;
    for (int t = 0; t < q_tokens; ++t) {
      const int v_flush = t / res_cap, tif = t % res_cap;
      const int64_t v_base = (int64_t)v_flush * num_heads_kv * res_cap * bpt +
                             (int64_t)kv_head * res_cap * bpt + (int64_t)tif * bpt;
      for (int b = 0; b < bpt; ++b) {
        oracle_kivi_dequantize_block(qv + (v_base + b) * bb, bits, buf);
        for (int i = 0; i < 32; ++i) oh[b * 32 + i] += w[t] * buf[i];
      }
    }
    for (int rt = 0; rt < res_tokens; ++rt) {
      const float *vp = res_v + (int64_t)kv_head * res_cap * head_dim + (int64_t)rt * head_dim;
      for (int d = 0; d < head_dim; ++d) oh[d] += w[q_tokens + rt] * vp[d];
    }
    free(w);
  }
  return 0;
}

/* ------------------------------------------------------------------------- */
/* a-4 score policy.                                                          */
/*   CPU producer: crates/techniques/attn-score/src/lib.rs begin_step 175-208,*/
/*   accumulate_layer_gqa 246-316, end_step 318-359 (flat + per-kv-head       */
/*   buffers only).                                                           */
/* ------------------------------------------------------------------------- */
ORACLE_API void oracle_score_begin_step(float *importance, float *head_importance,
                                        float *step_importance, float *head_step_importance,
                                        int max_seq_len, int n_kv_heads, float decay) {
  if (decay > 0.0f) {
    const float factor = 1.0f - decay;
    for (int i = 0; i < max_seq_len; ++i) importance[i] *= factor;
    for (int64_t i = 0; i < (int64_t)n_kv_heads * max_seq_len; ++i) head_importance[i] *= factor;
  }
  memset(step_importance, 0, sizeof(float) * (size_t)max_seq_len);
  memset(head_step_importance, 0, sizeof(float) * (size_t)n_kv_heads * max_seq_len);
}

ORACLE_API void oracle_score_accumulate_layer_gqa(const float *scores, int64_t stride,
                                                  int cache_seq_len, int n_heads_q,
                                                  int n_kv_heads, int score_offset,
                                                  float *step_importance,
                                                  float *head_step_importance, int max_seq_len) {
  const int len = cache_seq_len < max_seq_len ? cache_seq_len : max_seq_len;
  const int n_rep = n_heads_q / n_kv_heads;
  const float inv_rep = 1.0f / (float)n_rep;
  for (int t = 0; t < len; ++t) {
    const int pos = score_offset + t;
    if (pos >= max_seq_len) break;
    float layer_score = 0.0f;
    for (int h = 0; h < n_heads_q; ++h) layer_score += scores[h * stride + t];
    step_importance[pos] = fmaxf(step_importance[pos], layer_score);
    for (int kv = 0; kv < n_kv_heads; ++kv) {
      float g = 0.0f;
      for (int r = 0; r < n_rep; ++r) g += scores[(int64_t)(kv * n_rep + r) * stride + t];
      g *= inv_rep;
      const int64_t idx = (int64_t)kv * max_seq_len + pos;
      head_step_importance[idx] = fmaxf(head_step_importance[idx], g);
    }
  }
}

ORACLE_API void oracle_score_end_step(float *importance, float *head_importance,
                                      const float *step_importance,
                                      const float *head_step_importance, int max_seq_len,
                                      int n_kv_heads) {
  for (int t = 0; t < max_seq_len; ++t) importance[t] += step_importance[t];
  for (int64_t i = 0; i < (int64_t)n_kv_heads * max_seq_len; ++i)
    head_importance[i] += head_step_importance[i];
}

/* GPU reducer semantics: crates/techniques/attn-score/src/score_reduce.cu
 * kernel_score_fused_reduce 13-62, _per_layer 64-91. */
ORACLE_API int oracle_score_fused_reduce(const float *scores, float *importance,
                                         float *head_importance, float decay_factor,
                                         int n_layers, int n_heads_q, int n_kv_heads,
                                         int cache_seq_len, int64_t score_stride,
                                         int max_seq_len) {
  if (n_kv_heads <= 0 || n_kv_heads > 16) return -1;
  const int n_rep = n_heads_q / n_kv_heads;
  const float inv_rep = 1.0f / (float)n_rep;
  const int64_t layer_stride = (int64_t)n_heads_q * score_stride;
  for (int t = 0; t < cache_seq_len; ++t) {
    float step_flat = 0.0f, step_head[16] = {0};
    for (int l = 0; l < n_layers; ++l) {
      float layer_flat = 0.0f, layer_head[16] = {0};
      for (int h = 0; h < n_heads_q; ++h) {
        const float w = scores[l * layer_stride + h * score_stride + t];
        layer_flat += w;
        layer_head[h / n_rep] += w;
      }
      step_flat = fmaxf(step_flat, layer_flat);
      for (int kv = 0; kv < n_kv_heads; ++kv) step_head[kv] = fmaxf(step_head[kv], layer_head[kv] * inv_rep);
    }
    importance[t] = importance[t] * decay_factor + step_flat;
    for (int kv = 0; kv < n_kv_heads; ++kv) {
      const int64_t idx = (int64_t)kv * max_seq_len + t;
      head_importance[idx] = head_importance[idx] * decay_factor + step_head[kv];
    }
  }
  return 0;
}

ORACLE_API void oracle_score_reduce_per_layer(const float *scores, float *layer_flat,
                                              float decay_factor, int n_layers, int n_heads_q,
                                              int cache_seq_len, int64_t score_stride,
                                              int max_seq_len) {
  const int64_t layer_stride = (int64_t)n_heads_q * score_stride;
  for (int t = 0; t < cache_seq_len; ++t)
    for (int l = 0; l < n_layers; ++l) {
      float s = 0.0f;
      for (int h = 0; h < n_heads_q; ++h) s += scores[l * layer_stride + h * score_stride + t];
      const int64_t idx = (int64_t)l * max_seq_len + t;
      layer_flat[idx] = layer_flat[idx] * decay_factor + s;
    }
}

/* ------------------------------------------------------------------------- */
/* a-5 keep-list: compile_keep_top_k                                          */
/*   crates/argus-extension-api/src/lib.rs:788-810 (stable descending sort by */
/*   score, NaN compares Equal; ties keep position order).  Returns the       */
/*   keep-list length; `keep` must hold `current` entries.                    */
/* ------------------------------------------------------------------------- */
ORACLE_API int oracle_compile_keep_top_k(int current, int prefix, int recent, int heavy,
                                         const float *score, int32_t *keep) {
  if (prefix > current) prefix = current;
  int recent_start = current - recent;
  if (recent_start < 0) recent_start = 0;
  if (recent_start < prefix) recent_start = prefix;
  const int n_mid = recent_start - prefix;
  int n = 0;
  for (int i = 0; i < prefix; ++i) keep[n++] = i;
  if (heavy > 0 && n_mid > 0) {
    /* stable insertion-merge sort (Rust sort_by is a stable merge sort): any
     * stable sort with the same comparator yields the same order as long as
     * the comparator is a strict weak order; with NaN it is not, so NaN-free
     * scores are a precondition here. */
    int32_t *idx = (int32_t *)malloc(sizeof(int32_t) * (size_t)n_mid);
    int32_t *tmp = (int32_t *)malloc(sizeof(int32_t) * (size_t)n_mid);
    for (int i = 0; i < n_mid; ++i) idx[i] = prefix + i;
    for (int width = 1; width < n_mid; width *= 2) {
      for (int lo = 0; lo < n_mid; lo += 2 * width) {
        int mid = lo + width < n_mid ? lo + width : n_mid;
        int hi = lo + 2 * width < n_mid ? lo + 2 * width : n_mid;
        int a = lo, b = mid, o = lo;
        while (a < mid && b < hi) {
          /* take from the right run only if strictly greater score */
          const float sa = score ? score[idx[a]] : 0.0f, sb = score ? score[idx[b]] : 0.0f;
          if (sb > sa) tmp[o++] = idx[b++]; else tmp[o++] = idx[a++];
        }
        while (a < mid) tmp[o++] = idx[a++];
        while (b < hi) tmp[o++] = idx[b++];
      }
      int32_t *sw = idx; idx = tmp; tmp = sw;
    }
    const int take = heavy < n_mid ? heavy : n_mid;
    /* re-sort the taken positions ascending */
    for (int i = 1; i < take; ++i) {
      int32_t x = idx[i]; int j = i - 1;
      while (j >= 0 && idx[j] > x) { idx[j + 1] = idx[j]; --j; }
      idx[j + 1] = x;
    }
    for (int i = 0; i < take; ++i) keep[n++] = idx[i];
    free(idx); free(tmp);
  }
  for (int i = recent_start; i < current; ++i) keep[n++] = i;
  return n;
}

/* StreamingLLM keep_spec: crates/techniques/streaming-llm/src/lib.rs:27-62.
 * Returns -1 for None (within budget), else the keep-list length. */
ORACLE_API int oracle_streaming_keep(int sink_size, int window_size, int current, int target,
                                     int32_t *keep) {
  if (sink_size < 1) sink_size = 1;
  if (window_size < 1) window_size = 1;
  const int keep_n = sink_size + window_size;
  int eff = window_size;
  if (target > 0 && target < keep_n) {
    eff = target - sink_size;
    if (eff < 1) eff = 1;
  }
  if (current <= sink_size + eff) return -1;
  return oracle_compile_keep_top_k(current, sink_size, eff, 0, NULL, keep);
}

/* Compaction gather of kept rows to slots 0..n of a HeadMajor cache
 * (engine/src/kv/cache_handle.rs:154-210; independent model
 * engine/src/kv/naive_reference.rs:21-120).  elem_bytes = 2 (F16) or 4. */
ORACLE_API void oracle_compact_keep(const void *src, void *dst, const int32_t *keep, int n_keep,
                                    int kv_heads, int src_capacity, int dst_capacity,
                                    int head_dim, int elem_bytes) {
  const size_t row = (size_t)head_dim * elem_bytes;
  for (int h = 0; h < kv_heads; ++h)
    for (int i = 0; i < n_keep; ++i)
      memcpy((char *)dst + ((size_t)h * dst_capacity + i) * row,
             (const char *)src + ((size_t)h * src_capacity + keep[i]) * row, row);
}

/* ------------------------------------------------------------------------- */
/* f-1 KV write path: Backend::kv_scatter_f32_to_f16[_batch]                  */
/*   engine/src/backend.rs:425-545; device semantics                          */
/*   engine/src/backend/cuda_pc/kernels.cu:305-360.                           */
/*   src [seq_len, Hkv, d] F32 -> dst HeadMajor [Hkv, capacity, d].           */
/* ------------------------------------------------------------------------- */
ORACLE_API void oracle_kv_scatter(const float *k_src, const float *v_src, void *k_dst,
                                  void *v_dst, int kv_heads, int head_dim, int capacity,
                                  int write_pos_start, int seq_len, int dst_f16) {
  for (int s = 0; s < seq_len; ++s)
    for (int h = 0; h < kv_heads; ++h)
      for (int d = 0; d < head_dim; ++d) {
        const int64_t so = ((int64_t)s * kv_heads + h) * head_dim + d;
        const int64_t dofs = (int64_t)h * capacity * head_dim + (int64_t)(write_pos_start + s) * head_dim + d;
        if (dst_f16) {
          ((uint16_t *)k_dst)[dofs] = f2h(k_src[so]);
          ((uint16_t *)v_dst)[dofs] = f2h(v_src[so]);
        } else {
          ((float *)k_dst)[dofs] = k_src[so];
          ((float *)v_dst)[dofs] = v_src[so];
        }
      }
}

/* ---- PFA side channel ----------------------------------------------------------------------
 * prefill_attention_scores, engine/src/kv/standard_format.rs:1400-1510: for the trailing q_window
 * query rows of a prefill chunk, the post-softmax probability of every visible key, (a) summed
 * over the rows into sum_out[h][key] (+=) and/or (b) per row: per_head -> out[step][h][key] = p,
 * else out[step][key] += p / n_heads_q.  Scalar f32 dot (mul then add), logit = dot * scale,
 * row maximum, e = exp(logit - max), denom summed in key order, p = e / denom.  K is F32 with the
 * caller's strides (elements).  window < 0 means no window; lo = p - (window - 1), saturating. */
ORACLE_API int oracle_prefill_attention_scores(const float *q, const float *k, int n_heads_q,
                                               int n_heads_kv, int head_dim, int seq_len,
                                               int cache_seq_len, int64_t k_pos_stride,
                                               int64_t kv_head_stride, int q_start_pos, int q_window,
                                               int window, float *sum_out, float *per_row_out,
                                               int per_row_per_head) {
  if (n_heads_kv <= 0 || n_heads_q % n_heads_kv) return -1;
  const int prefix_len = cache_seq_len;
  const float scale = 1.0f / sqrtf((float)head_dim);
  const int gqa = n_heads_q / n_heads_kv;
  const int64_t q_row_stride = (int64_t)n_heads_q * head_dim;
  const int qwin = q_window < seq_len ? q_window : seq_len;
  const int qwin_start = seq_len - qwin;
  const float inv_heads = 1.0f / (float)n_heads_q;
  float *scratch = (float *)malloc(sizeof(float) * (size_t)(prefix_len > 0 ? prefix_len : 1));
  if (!scratch) return -2;
  for (int h = 0; h < n_heads_q; ++h) {
    const int kv_head = h / gqa;
    const int64_t out_row_base = (int64_t)h * prefix_len;
    for (int r = qwin_start; r < seq_len; ++r) {
      const int p = q_start_pos + r;
      int lo = 0;
      if (window >= 0) {
        const int w1 = window > 0 ? window - 1 : 0;
        lo = p > w1 ? p - w1 : 0;
      }
      const float *qv = q + (int64_t)r * q_row_stride + (int64_t)h * head_dim;
      float maxv = -INFINITY;
      for (int key = lo; key <= p; ++key) {
        const float *kv = k + (int64_t)key * k_pos_stride + (int64_t)kv_head * kv_head_stride;
        float dot = 0.0f;
        for (int d = 0; d < head_dim; ++d) dot += qv[d] * kv[d];
        const float logit = dot * scale;
        scratch[key] = logit;
        if (logit > maxv) maxv = logit;
      }
      float denom = 0.0f;
      for (int key = lo; key <= p; ++key) {
        const float e = expf(scratch[key] - maxv);
        scratch[key] = e;
        denom += e;
      }
      if (sum_out)
        for (int key = lo; key <= p; ++key) sum_out[out_row_base + key] += scratch[key] / denom;
      if (per_row_out) {
        const int step = r - qwin_start;
        if (per_row_per_head) {
          float *dst = per_row_out + (int64_t)step * n_heads_q * prefix_len + out_row_base;
          for (int key = lo; key <= p; ++key) dst[key] = scratch[key] / denom;
        } else {
          float *dst = per_row_out + (int64_t)step * prefix_len;
          for (int key = lo; key <= p; ++key) dst[key] += (scratch[key] / denom) * inv_heads;
        }
      }
    }
  }
  free(scratch);
  return 0;
}

/* ---- descriptor-driven block formats (--kv-format floor) ---------------------------------------
 * unpack_block_via_descriptor / decode_via_descriptor, engine/src/format/dtype_layout.rs:102-166,
 * 285-300, and encode_via_descriptor with its two canonical encoders, 302-396.
 * scale_layout: 0 None, 1 PerBlockF16, 2 PerBlockF16WithMin; packing: 0 Dense, 1 Nibble, 2 Byte,
 * 3 Quad (argus-extension-api lib.rs:1111-1138).  Block = [f16 scale][f16 min?][packed quants]. */
static int desc_block_bytes(int block_elems, int scale_layout, int packing) {
  int q;
  switch (packing) {
    case 1: q = block_elems / 2; break;
    case 2: q = block_elems; break;
    case 3: q = block_elems / 4; break;
    default: return -1;
  }
  return q + (scale_layout == 1 ? 2 : scale_layout == 2 ? 4 : 0);
}

ORACLE_API int oracle_desc_block_bytes(int block_elems, int scale_layout, int packing) {
  return desc_block_bytes(block_elems, scale_layout, packing);
}

ORACLE_API int oracle_decode_via_descriptor(int block_elems, int bits, int scale_layout, int packing,
                                            const uint8_t *src, float *dst, int64_t n_elems) {
  const int bb = desc_block_bytes(block_elems, scale_layout, packing);
  if (bb <= 0 || block_elems <= 0 || n_elems % block_elems) return -1;
  const int n = block_elems;
  for (int64_t bi = 0; bi < n_elems / n; ++bi) {
    const uint8_t *block = src + bi * bb;
    float *out = dst + bi * n;
    uint16_t sb, mb = 0;
    memcpy(&sb, block, 2);
    const float scale = h2f(sb);
    float min = 0.0f;
    const uint8_t *quants = block + 2;
    if (scale_layout == 2) {
      memcpy(&mb, block + 2, 2);
      min = h2f(mb);
      quants = block + 4;
    }
    if (packing == 1) {
      const int half = n / 2, is_signed = scale_layout == 1, zp = 1 << (bits - 1);
      for (int i = 0; i < half; ++i) {
        const int lo = quants[i] & 0x0f, hi = quants[i] >> 4;
        if (is_signed) {
          out[i] = (float)(lo - zp) * scale;
          out[i + half] = (float)(hi - zp) * scale;
        } else {
          out[i] = (float)lo * scale + min;
          out[i + half] = (float)hi * scale + min;
        }
      }
    } else if (packing == 2) {
      for (int i = 0; i < n; ++i) out[i] = (float)(int)(int8_t)quants[i] * scale;
    } else {
      for (int i = 0; i < n / 4; ++i)
        for (int j = 0; j < 4; ++j) out[i * 4 + j] = (float)((quants[i] >> (j * 2)) & 3) * scale + min;
    }
  }
  return 0;
}

ORACLE_API int oracle_encode_via_descriptor(int block_elems, int bits, int scale_layout, int packing,
                                            const float *src, uint8_t *dst, int64_t n_elems) {
  const int quad = (scale_layout == 2 && packing == 3);
  if (!quad && !(scale_layout == 1 && packing == 1)) return -2;  /* outside the writable floor */
  const int bb = desc_block_bytes(block_elems, scale_layout, packing);
  if (block_elems <= 0 || n_elems % block_elems) return -1;
  const int n = block_elems;
  for (int64_t bi = 0; bi < n_elems / n; ++bi) {
    const float *s = src + bi * n;
    uint8_t *d8 = dst + bi * bb;
    if (!quad) {
      const float qmax = (float)((1 << (bits - 1)) - 1), qmin = -(float)(1 << (bits - 1));
      const int zp = 1 << (bits - 1), half = n / 2;
      float max_abs = 0.0f;
      for (int i = 0; i < n; ++i) max_abs = fmaxf(max_abs, fabsf(s[i]));  /* f32::max ignores NaN like fmaxf */
      const float d = max_abs / qmax;
      const float id = d == 0.0f ? 0.0f : 1.0f / d;
      const uint16_t db = f2h(d);
      memcpy(d8, &db, 2);
      for (int i = 0; i < half; ++i) {
        const int v0 = (int)fminf(fmaxf(roundf(s[i] * id), qmin), qmax);
        const int v1 = (int)fminf(fmaxf(roundf(s[i + half] * id), qmin), qmax);
        d8[2 + i] = (uint8_t)((uint8_t)(v0 + zp) | ((uint8_t)(v1 + zp) << 4));
      }
    } else {
      const float qmax = (float)((1u << bits) - 1u);
      const int per_byte = 8 / bits;
      float mn = INFINITY, mx = -INFINITY;
      for (int i = 0; i < n; ++i) {
        mn = fminf(mn, s[i]);
        mx = fmaxf(mx, s[i]);
      }
      const float d = (mx - mn) / qmax;
      const float id = d == 0.0f ? 0.0f : 1.0f / d;
      const uint16_t db = f2h(d), mb = f2h(mn);
      memcpy(d8, &db, 2);
      memcpy(d8 + 2, &mb, 2);
      for (int i = 0; i < n / per_byte; ++i) {
        uint8_t byte = 0;
        for (int j = 0; j < per_byte; ++j) {
          const uint8_t qv = (uint8_t)fminf(fmaxf(roundf((s[i * per_byte + j] - mn) * id), 0.0f), qmax);
          byte |= (uint8_t)(qv << (j * bits));
        }
        d8[4 + i] = byte;
      }
    }
  }
  return 0;
}
