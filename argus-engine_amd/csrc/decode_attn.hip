// Split-KV flash-decode for single-query GQA attention on gfx950.
//
// Stands in for Backend::attention_gen (engine/src/backend.rs:284-295; CPU semantics
// engine/src/backend/cpu/x86.rs:178-357 and common.rs:359-675).
//
// Design (HBM-bound: every K/V byte is read exactly once per call):
//  * One workgroup (4 waves) owns one (sequence, KV head, KV split).  All Hq/Hkv query heads of
//    the group share the single pass over K and V, so GQA does not multiply traffic.
//  * A wave reads K/V rows with 16-byte loads; LPR = row_bytes/16 consecutive lanes cover one
//    row, so each load instruction of a wave covers 64/LPR whole rows = 1 KiB of contiguous
//    memory.  U such loads for K and U for V are in flight per wave before any use.
//  * q.k partial sums are reduced over the LPR lanes with DPP adds (no LDS); afterwards every
//    lane of a row group holds that row's logit, which is exactly the weight it needs for its
//    slice of the V row.  Each row group keeps a private online-softmax state (m, l, acc) that is
//    merged once at the end: shuffles across row groups, LDS across the 4 waves.
//  * Each workgroup writes one partial (m, l, un-normalised out) per Q head; a second kernel
//    combines the splits with a log-sum-exp merge, writes `out`, and -- when post-softmax scores
//    were requested -- turns the logits the first pass stored in `scores_out` into probabilities
//    in place (exact global max / sum are only known there).
#include "decode_common.hpp"

#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <type_traits>

namespace {

using namespace argus_decode;

template <typename KV_T>
struct KvVec;
template <>
struct KvVec<_Float16> {
  static constexpr int E = 8;
  using vec = half8_t;
};
template <>
struct KvVec<float> {
  static constexpr int E = 4;
  using vec = float4_t;
};
// Descriptor-driven rows: a lane decodes 8 consecutive channels of its row's block.
typedef float float8_t __attribute__((ext_vector_type(8)));
template <>
struct KvVec<DescRow> {
  static constexpr int E = 8;
  using vec = float8_t;
};

// The lane's piece (E channels from c0) of the row in `slot` of one KV head.
template <typename KV_T>
__device__ __forceinline__ typename KvVec<KV_T>::vec load_row_piece(const DecodeParams &p, const void *cache, int64_t head_elem, int64_t slot,
                                                                     int c0) {
  using vec_t = typename KvVec<KV_T>::vec;
  if constexpr (std::is_same<KV_T, DescRow>::value) {
    const int64_t elem = head_elem + slot * p.row_stride + c0;
    float v[8];
    desc_decode8(p, (const uint8_t *)cache + desc_block_offset(p, elem), (int)(elem % p.desc_block_elems), v);
    return float8_t{v[0], v[1], v[2], v[3], v[4], v[5], v[6], v[7]};
  } else {
    return __builtin_nontemporal_load((const vec_t *)((const KV_T *)cache + head_elem + slot * p.row_stride + c0));
  }
}

enum DecodeMode { kPlain = 0, kSoftcap = 1, kGeneric = 2 };

template <int D, int GT, typename KV_T, int U, int MODE>
__global__ __launch_bounds__(256) void decode_split_kernel(const DecodeParams p) {
  constexpr int E = KvVec<KV_T>::E;
  using vec_t = typename KvVec<KV_T>::vec;
  constexpr int LPR = D / E;       // lanes per K/V row
  constexpr int RPW = 64 / LPR;    // rows per wave load instruction
  constexpr int TILE = RPW * U;    // rows per wave iteration
  static_assert(LPR >= GT && LPR <= 64, "row group must cover the query-head tile");

  // A GQA group wider than the head tile is covered by several workgroups per KV head, GT heads each
  // (they re-read the KV rows: this kernel is the fall-back for such shapes, not their fast path).
  const int split = blockIdx.x, kvh = blockIdx.y / p.head_chunks, b = blockIdx.z;
  const int hchunk = blockIdx.y % p.head_chunks;
  const int hbase = kvh * p.group + GT * hchunk;        // first query head of this workgroup
  const int gcount = min(GT, p.group - GT * hchunk);    // and how many it has
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int grp = lane / LPR, sub = lane % LPR;
  const int c0 = sub * E;

  const int t_begin = split * p.chunk;
  const int t_end = min(p.len, t_begin + p.chunk);

  const int64_t head_elem = (int64_t)b * p.kv_bs + (int64_t)kvh * p.head_stride;  // first element of this KV head's rows
  const int32_t *idx = p.kv_index ? p.kv_index + (int64_t)b * p.index_bs : nullptr;

  // This lane's slice of every query head of the group (heads beyond the group are clamped
  // duplicates whose results are never written).
  float q[GT][E];
#pragma unroll
  for (int g = 0; g < GT; ++g) {
    const int h = hbase + min(g, gcount - 1);
    const float *qp = p.q + (int64_t)b * p.q_bs + (int64_t)h * D + c0;
#pragma unroll
    for (int e = 0; e < E; ++e) q[g][e] = qp[e] * p.scale;
  }

  float m[GT], l[GT], acc[GT][E];
#pragma unroll
  for (int g = 0; g < GT; ++g) {
    m[g] = kNegInf;
    l[g] = 0.0f;
#pragma unroll
    for (int e = 0; e < E; ++e) acc[g][e] = 0.0f;
  }

  const bool use_idx = (MODE == kGeneric) && idx != nullptr;
  const bool use_cap = (MODE == kSoftcap) || (MODE == kGeneric && p.softcap > 0.0f);
  const float inv_cap = use_cap ? 1.0f / p.softcap : 0.0f;

  // One tile = U load instructions per stream per wave.  FULL tiles need no row masking.
  auto process_tile = [&](const int base, auto full_tag) {
    constexpr bool FULL = decltype(full_tag)::value;
    vec_t kr[U], vr[U];
    bool valid[U];
    int64_t slot[U];
    int tc[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int t = base + u * RPW + grp;
      valid[u] = FULL || t < t_end;
      tc[u] = valid[u] ? t : (t_end - 1);
    }
    if (use_idx) {  // uniform
      // The list entries of all U rows are requested together and before the rows: read one by one
      // between the rows, every entry's wait also waited for the rows requested before it.
      uint32_t entry[U];
#pragma unroll
      for (int u = 0; u < U; ++u) entry[u] = (uint32_t)idx[tc[u]];
      // a slot outside the cache (stale or negative list entry) is clamped to the last one: the rows
      // are fetched with plain loads, which nothing else bounds
#pragma unroll
      for (int u = 0; u < U; ++u) slot[u] = (int64_t)min(entry[u], (uint32_t)(p.slot_bound - 1));
    } else {
#pragma unroll
      for (int u = 0; u < U; ++u) slot[u] = (int64_t)(p.kv_start + tc[u]);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      kr[u] = load_row_piece<KV_T>(p, p.k, head_elem, slot[u], c0);
      vr[u] = load_row_piece<KV_T>(p, p.v, head_elem, slot[u], c0);
    }

    float s[U][GT];
#pragma unroll
    for (int u = 0; u < U; ++u) {
#pragma unroll
      for (int g = 0; g < GT; ++g) {
        float part = 0.0f;
#pragma unroll
        for (int e = 0; e < E; ++e) part = fmaf(q[g][e], (float)kr[u][e], part);
        float sv = group_allreduce_sum<LPR>(part);
        // NaN logit counts as -inf (common.rs:555-560)
        if (use_cap) {
          const float capped = softcap_tanh(sv, p.softcap, inv_cap);
          sv = (sv != sv) ? kNegInf : capped;
        } else {
          sv = fmaxf(sv, kNegInf);
        }
        s[u][g] = valid[u] ? sv : kNegInf;
      }
    }

    if (p.scores) {
      // Store the logits; the combine pass rewrites them as probabilities.
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int t = base + u * RPW + grp;
#pragma unroll
        for (int g = 0; g < GT; ++g) {
          if (sub == g && g < gcount && valid[u])
            __builtin_nontemporal_store(s[u][g], p.scores + (int64_t)b * p.score_bs + (int64_t)(hbase + g) * p.score_stride + t);
        }
      }
    }

#pragma unroll
    for (int g = 0; g < GT; ++g) {
      float mt = s[0][g];
#pragma unroll
      for (int u = 1; u < U; ++u) mt = fmaxf(mt, s[u][g]);
      const float m_new = fmaxf(m[g], mt);
      const float m_ref = (m_new == kNegInf) ? 0.0f : m_new;
      const float alpha = __expf(m[g] - m_ref);
      m[g] = m_new;
      float lsum = 0.0f;
#pragma unroll
      for (int e = 0; e < E; ++e) acc[g][e] *= alpha;
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const float pw = __expf(s[u][g] - m_ref);
        lsum += pw;
#pragma unroll
        for (int e = 0; e < E; ++e) acc[g][e] = fmaf(pw, (float)vr[u][e], acc[g][e]);
      }
      l[g] = l[g] * alpha + lsum;
    }
  };

  {
    int base = t_begin + wave * TILE;
    for (; base + TILE <= t_end; base += 4 * TILE) process_tile(base, std::true_type{});
    if (base < t_end) process_tile(base, std::false_type{});
  }

  // ---- merge the RPW row groups of this wave --------------------------------------------
#pragma unroll
  for (int g = 0; g < GT; ++g) {
    float mw = m[g];
#pragma unroll
    for (int off = LPR; off < 64; off <<= 1) mw = fmaxf(mw, __shfl_xor(mw, off, 64));
    const float m_ref = (mw == kNegInf) ? 0.0f : mw;
    const float f = __expf(m[g] - m_ref);
    float lw = l[g] * f;
#pragma unroll
    for (int off = LPR; off < 64; off <<= 1) lw += __shfl_xor(lw, off, 64);
#pragma unroll
    for (int e = 0; e < E; ++e) {
      float a = acc[g][e] * f;
#pragma unroll
      for (int off = LPR; off < 64; off <<= 1) a += __shfl_xor(a, off, 64);
      acc[g][e] = a;
    }
    m[g] = mw;
    l[g] = lw;
  }

  // ---- merge the 4 waves through LDS ------------------------------------------------------
  __shared__ float lds_m[4][GT], lds_l[4][GT];
  __shared__ float lds_acc[4][GT][D];
  if (grp == 0) {
#pragma unroll
    for (int g = 0; g < GT; ++g) {
      if (sub == 0) {
        lds_m[wave][g] = m[g];
        lds_l[wave][g] = l[g];
      }
#pragma unroll
      for (int e = 0; e < E; ++e) lds_acc[wave][g][c0 + e] = acc[g][e];
    }
  }
  __syncthreads();

  for (int i = threadIdx.x; i < gcount * D; i += 256) {
    const int g = i / D, c = i % D;
    const int h = hbase + g;
    float mm = fmaxf(fmaxf(lds_m[0][g], lds_m[1][g]), fmaxf(lds_m[2][g], lds_m[3][g]));
    const float m_ref = (mm == kNegInf) ? 0.0f : mm;
    float o = 0.0f, ll = 0.0f;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      const float f = __expf(lds_m[w][g] - m_ref);
      o += lds_acc[w][g][c] * f;
      ll += lds_l[w][g] * f;
    }
    if (p.direct) {
      // Single split, no scores: finish here.  A row without any finite logit is left to the
      // fallback below.
      if (ll > 0.0f && ll < __builtin_huge_valf()) p.out[(int64_t)b * p.out_bs + (int64_t)h * D + c] = o / ll;
    } else {
      const int64_t pidx = ((int64_t)b * p.n_heads_q + h) * p.nsplit + split;
      p.ws_o[pidx * D + c] = o;
      if (c == 0) {
        p.ws_ml[pidx * 2 + 0] = mm;
        p.ws_ml[pidx * 2 + 1] = ll;
      }
    }
  }
  if (p.direct) {
    for (int g = 0; g < gcount; ++g) {
      const float mm = fmaxf(fmaxf(lds_m[0][g], lds_m[1][g]), fmaxf(lds_m[2][g], lds_m[3][g]));
      const float m_ref = (mm == kNegInf) ? 0.0f : mm;
      float ll = 0.0f;
      for (int w = 0; w < 4; ++w) ll += lds_l[w][g] * __expf(lds_m[w][g] - m_ref);
      if (!(ll > 0.0f && ll < __builtin_huge_valf())) uniform_fallback<KV_T>(p, b, hbase + g, D);
    }
  }
}

template <int D, int GT, typename KV_T>
constexpr int unroll_for() {
  // Keep q + acc + in-flight K/V rows inside the register file at >= 2 waves per SIMD.
  if (std::is_same<KV_T, DescRow>::value) return GT >= 4 ? 1 : 2;  // decoded rows are 8 floats per piece
  return GT >= 8 ? 2 : (GT >= 4 ? 4 : 8);
}

template <int D, int GT, typename KV_T>
int launch_decode(argus_hip_ctx *ctx, DecodeParams &p, int batch, bool want_scores, hipStream_t stream) {
  constexpr int U = unroll_for<D, GT, KV_T>();
  constexpr int E = KvVec<KV_T>::E;
  constexpr int tile_rows = 4 * (64 / (D / E)) * U;  // rows one workgroup consumes per iteration

  p.head_chunks = (p.group + GT - 1) / GT;
  const int pairs = batch * p.n_heads_kv * p.head_chunks;
  // Many more workgroups than resident slots, so the last partially filled round of the grid
  // costs little; bounded below by one tile per wave.
  const int target_wgs = ctx->compute_units * 24;
  const int max_splits = (p.len + tile_rows - 1) / tile_rows;
  int nsplit = std::max(1, std::min({(target_wgs + pairs - 1) / pairs, max_splits, kMaxSplits}));
  int chunk = (p.len + nsplit - 1) / nsplit;
  chunk = (chunk + tile_rows - 1) / tile_rows * tile_rows;
  nsplit = (p.len + chunk - 1) / chunk;
  p.chunk = chunk;
  p.nsplit = nsplit;
  p.direct = (nsplit == 1 && !want_scores) ? 1 : 0;

  if (!p.direct) {
    const int rc = reserve_partials(ctx, p, batch, D);
    if (rc != ARGUS_HIP_OK) return rc;
  }
  ctx->plan = argus_hip_decode_plan{nsplit, chunk, 0, 0, p.direct ? 1 : 2, 0, 0};

  dim3 grid(nsplit, p.n_heads_kv * p.head_chunks, batch);
  KernelTimer timer(ctx, stream);
  if (p.kv_index)
    hipLaunchKernelGGL((decode_split_kernel<D, GT, KV_T, U, kGeneric>), grid, dim3(256), 0, stream, p);
  else if (p.softcap > 0.0f)
    hipLaunchKernelGGL((decode_split_kernel<D, GT, KV_T, U, kSoftcap>), grid, dim3(256), 0, stream, p);
  else
    hipLaunchKernelGGL((decode_split_kernel<D, GT, KV_T, U, kPlain>), grid, dim3(256), 0, stream, p);
  timer.mark();
  ARGUS_HIP_CHECK(ctx, hipGetLastError());
  if (!p.direct) {
    hipLaunchKernelGGL((decode_combine_kernel<UniformFallback<KV_T>, D>), combine_grid(p, batch), dim3(256), 0, stream, p);
    ARGUS_HIP_CHECK(ctx, hipGetLastError());
  }
  return ARGUS_HIP_OK;
}

template <int D, typename KV_T>
int dispatch_group(argus_hip_ctx *ctx, DecodeParams &p, int batch, bool want_scores, hipStream_t stream) {
  if (p.group <= 1) return launch_decode<D, 1, KV_T>(ctx, p, batch, want_scores, stream);
  if (p.group <= 2) return launch_decode<D, 2, KV_T>(ctx, p, batch, want_scores, stream);
  if (p.group <= 4) return launch_decode<D, 4, KV_T>(ctx, p, batch, want_scores, stream);
  return launch_decode<D, 8, KV_T>(ctx, p, batch, want_scores, stream);  // wider groups: several head tiles per KV head
}

template <typename KV_T>
int dispatch_dim(argus_hip_ctx *ctx, DecodeParams &p, int D, int batch, bool want_scores, hipStream_t stream) {
  switch (D) {
    case 64: return dispatch_group<64, KV_T>(ctx, p, batch, want_scores, stream);
    case 128: return dispatch_group<128, KV_T>(ctx, p, batch, want_scores, stream);
    case 256: return dispatch_group<256, KV_T>(ctx, p, batch, want_scores, stream);
    default: return argus_fail(ctx, ARGUS_HIP_ERR_UNSUPPORTED, "head_dim %d not in {64,128,256}", D);
  }
}

}  // namespace

// kv_dtype value used internally for rows described by `desc`
constexpr int kKvDesc = 100;

static int attention_gen_impl(argus_hip_ctx *ctx, const argus_hip_attention_gen_args *a, int kv_dtype,
                              const argus_hip_kv_layout_desc *desc, int desc_block_bytes) {
  if (!ctx || !a) return ARGUS_HIP_ERR_INVALID;
  if (!a->q || !a->k_cache || !a->v_cache || !a->out)
    return argus_fail(ctx, ARGUS_HIP_ERR_INVALID, "attention_gen: null tensor pointer");
  if (a->num_heads_q <= 0 || a->num_heads_kv <= 0 || a->num_heads_q % a->num_heads_kv)
    return argus_fail(ctx, ARGUS_HIP_ERR_INVALID, "attention_gen: heads %d/%d", a->num_heads_q, a->num_heads_kv);
  if (a->cache_seq_len <= 0 || a->batch <= 0 || a->kv_start < 0)
    return argus_fail(ctx, ARGUS_HIP_ERR_INVALID, "attention_gen: cache_seq_len %d batch %d kv_start %d",
                      a->cache_seq_len, a->batch, a->kv_start);
  if (a->layout != ARGUS_HIP_HEAD_MAJOR && a->layout != ARGUS_HIP_SEQ_MAJOR)
    return argus_fail(ctx, ARGUS_HIP_ERR_INVALID, "attention_gen: layout %d", a->layout);
  if (a->layout == ARGUS_HIP_HEAD_MAJOR && !a->kv_index && a->kv_start + a->cache_seq_len > a->capacity)
    return argus_fail(ctx, ARGUS_HIP_ERR_INVALID, "attention_gen: kv_start %d + len %d exceeds capacity %d",
                      a->kv_start, a->cache_seq_len, a->capacity);
  if (a->scores_out && a->score_stride < a->cache_seq_len)
    return argus_fail(ctx, ARGUS_HIP_ERR_INVALID, "attention_gen: score_stride %d < cache_seq_len %d",
                      a->score_stride, a->cache_seq_len);
  if (a->score_stats && !a->scores_out)
    return argus_fail(ctx, ARGUS_HIP_ERR_INVALID, "attention_gen: score_stats without scores_out");
  if (a->batch > 65535 || a->num_heads_kv > 65535)
    return argus_fail(ctx, ARGUS_HIP_ERR_UNSUPPORTED, "attention_gen: batch / kv heads beyond grid limits");

  const int D = a->head_dim;
  if (D != 64 && D != 128 && D != 256)
    return argus_fail(ctx, ARGUS_HIP_ERR_UNSUPPORTED, "attention_gen: head_dim %d not in {64,128,256}", D);
  // An index list names slots of a HeadMajor cache of `capacity` rows (of the `capacity` first
  // positions of a SeqMajor one); a slot outside [0, capacity) never reaches memory outside the head's rows -- the vector-ALU kernel
  // clamps it to the last slot, the matrix-core kernels read it as a row of zeros -- and the result
  // for such a list is unspecified (the host mirror's attention_into_selected rejects it up front).
  if (a->kv_index && a->capacity <= 0)
    return argus_fail(ctx, ARGUS_HIP_ERR_INVALID, "attention_gen: kv_index needs capacity > 0 (got %d)", a->capacity);
  DecodeParams p{};
  p.q = a->q;
  p.k = a->k_cache;
  p.v = a->v_cache;
  p.out = a->out;
  p.scores = a->scores_out;
  p.score_stats = a->score_stats;
  p.stats_bs = a->stats_batch_stride ? a->stats_batch_stride : (int64_t)a->num_heads_q * 2;
  p.kv_index = a->kv_index;
  p.n_heads_q = a->num_heads_q;
  p.n_heads_kv = a->num_heads_kv;
  p.group = a->num_heads_q / a->num_heads_kv;
  p.len = a->cache_seq_len;
  p.kv_start = a->kv_index ? 0 : a->kv_start;
  p.slot_bound = a->capacity;
  p.score_stride = a->score_stride;
  if (a->layout == ARGUS_HIP_HEAD_MAJOR) {
    p.row_stride = D;
    p.head_stride = (int64_t)a->capacity * D;
  } else {
    p.row_stride = (int64_t)a->num_heads_kv * D;
    p.head_stride = D;
  }
  p.q_bs = a->q_batch_stride ? a->q_batch_stride : (int64_t)a->num_heads_q * D;
  p.out_bs = a->out_batch_stride ? a->out_batch_stride : (int64_t)a->num_heads_q * D;
  p.kv_bs = a->kv_batch_stride;
  p.score_bs = a->score_batch_stride ? a->score_batch_stride : (int64_t)a->num_heads_q * a->score_stride;
  p.index_bs = a->index_batch_stride;
  p.scale = a->scale != 0.0f ? a->scale : 1.0f / sqrtf((float)D);
  p.softcap = a->softcap;
  if (a->batch > 1 && p.kv_bs == 0)
    return argus_fail(ctx, ARGUS_HIP_ERR_INVALID, "attention_gen: batch > 1 needs kv_batch_stride");
  // The kernels move K/V rows and output rows as 16-byte vectors.
  const bool blocks = kv_dtype == ARGUS_HIP_Q4_0 || kv_dtype == ARGUS_HIP_Q4_1 || kv_dtype == ARGUS_HIP_Q8_0 || kv_dtype == ARGUS_HIP_Q2_0;
  const int64_t kv_vec = kv_dtype == kKvDesc ? desc->block_elems : blocks ? 32 : (kv_dtype == ARGUS_HIP_F16 ? 8 : 4);
  if (kv_dtype == kKvDesc) {
    p.desc_block_elems = (int32_t)desc->block_elems;
    p.desc_bits = desc->bits;
    p.desc_scale_layout = (int32_t)desc->scale_layout;
    p.desc_packing = (int32_t)desc->packing;
    p.desc_block_bytes = desc_block_bytes;
    // rows are whole blocks; blocks are read as 16-bit units
    if ((p.row_stride % kv_vec) || (p.head_stride % kv_vec) || (((uintptr_t)a->k_cache | (uintptr_t)a->v_cache) & 1) || ((uintptr_t)a->out & 15))
      return argus_fail(ctx, ARGUS_HIP_ERR_INVALID, "attention_gen_desc: strides must be whole blocks, caches 2-byte and out 16-byte aligned");
  } else if (((uintptr_t)a->k_cache | (uintptr_t)a->v_cache | (uintptr_t)a->out) & 15)
    return argus_fail(ctx, ARGUS_HIP_ERR_INVALID, "attention_gen: k/v/out must be 16-byte aligned");
  if ((p.kv_bs % kv_vec) || (p.out_bs % 4))
    return argus_fail(ctx, ARGUS_HIP_ERR_INVALID, "attention_gen: batch strides must keep 16-byte alignment");

  hipStream_t stream = (hipStream_t)a->stream;
  const bool want_scores = a->scores_out != nullptr;
  // ARGUS_HIP_DECODE=valu (read when the context is created) keeps the vector-ALU kernel for A/B measurements.
  const bool force_valu = ctx->env.decode_valu;
  if (blocks && p.len < 64 && (p.row_stride % 32) == 0 && (p.head_stride % 32) == 0) {
    // A handful of tokens gives the f16 roundings of the matrix-core kernel's weights nothing to
    // average out against (q2_0 rows of 3 tokens with values near 8: 2.1-2.2e-3 in a seeded sweep,
    // bar 2e-3); such rows cost nothing either way and take the vector-ALU kernel, which decodes the
    // same blocks through their descriptor and works in f32, as F16 rows of this length do.
    p.desc_block_elems = 32;
    p.desc_bits = kv_dtype == ARGUS_HIP_Q8_0 ? 8 : kv_dtype == ARGUS_HIP_Q2_0 ? 2 : 4;
    p.desc_scale_layout = (kv_dtype == ARGUS_HIP_Q4_1 || kv_dtype == ARGUS_HIP_Q2_0) ? 2 : 1;  // PerBlockF16WithMin : PerBlockF16
    p.desc_packing = kv_dtype == ARGUS_HIP_Q8_0 ? 2 : kv_dtype == ARGUS_HIP_Q2_0 ? 3 : 1;     // Byte : Quad : Nibble
    p.desc_block_bytes = kv_dtype == ARGUS_HIP_Q8_0 ? 34 : kv_dtype == ARGUS_HIP_Q2_0 ? 12 : kv_dtype == ARGUS_HIP_Q4_1 ? 20 : 18;
    return dispatch_dim<DescRow>(ctx, p, D, a->batch, want_scores, stream);
  }
  if (blocks) return launch_decode_blocks(ctx, p, D, kv_dtype, a->batch, stream);
  if (!force_valu && decode_mfma_supported(p, D, kv_dtype, a->batch)) return launch_decode_mfma(ctx, p, D, a->batch, stream);
  switch (kv_dtype) {
    case ARGUS_HIP_F16: return dispatch_dim<_Float16>(ctx, p, D, a->batch, want_scores, stream);
    case ARGUS_HIP_F32: return dispatch_dim<float>(ctx, p, D, a->batch, want_scores, stream);
    case kKvDesc: return dispatch_dim<DescRow>(ctx, p, D, a->batch, want_scores, stream);
    default: return argus_fail(ctx, ARGUS_HIP_ERR_UNSUPPORTED, "attention_gen: kv dtype %d", kv_dtype);
  }
}

ARGUS_API int argus_hip_attention_gen(argus_hip_ctx *ctx, const argus_hip_attention_gen_args *a) {
  if (!ctx || !a) return ARGUS_HIP_ERR_INVALID;
  return attention_gen_impl(ctx, a, a->kv_dtype, nullptr, 0);
}

// attention_gen over a cache whose rows are blocks of any descriptor the generic floor decodes
// (PerBlockF16 / PerBlockF16WithMin x Nibble / Byte / Quad, block_elems a multiple of 8 up to 64 that
// divides head_dim).  The four named 32-element formats go to the matrix-core block kernel; every
// other one is attended by the vector-ALU kernel, each lane decoding the 8 channels of its piece from
// the row's blocks.  Anything else is declined with ARGUS_HIP_ERR_UNSUPPORTED (nothing launched), which
// is the caller's cue to take the floor: decode the cache with argus_hip_kv_decode_descriptor (or on
// the CPU) and attend the F16 / F32 copy.
ARGUS_API int argus_hip_attention_gen_desc(argus_hip_ctx *ctx, const argus_hip_attention_gen_args *a, const argus_hip_kv_layout_desc *d) {
  if (!ctx || !a || !d) return ARGUS_HIP_ERR_INVALID;
  int q;
  switch (d->packing) {
    case 1: q = (int)d->block_elems / 2; break;
    case 2: q = (int)d->block_elems; break;
    case 3: q = (int)d->block_elems / 4; break;
    default: return argus_fail(ctx, ARGUS_HIP_ERR_UNSUPPORTED, "attention_gen_desc: declined, packing %u has no block form", d->packing);
  }
  if (d->scale_layout != 1 && d->scale_layout != 2)
    return argus_fail(ctx, ARGUS_HIP_ERR_UNSUPPORTED, "attention_gen_desc: declined, scale layout %u", d->scale_layout);
  const bool bits_ok = (d->packing == 1 && d->bits >= 2 && d->bits <= 4) || (d->packing == 2 && d->bits == 8) || (d->packing == 3 && d->bits == 2);
  if (!bits_ok || d->block_elems == 0 || d->block_elems > 64 || d->block_elems % 8 || (d->packing == 3 && d->scale_layout != 2))
    return argus_fail(ctx, ARGUS_HIP_ERR_UNSUPPORTED, "attention_gen_desc: declined, block_elems %u bits %u", d->block_elems, (unsigned)d->bits);
  if (a->head_dim <= 0 || a->head_dim % (int)d->block_elems)
    return argus_fail(ctx, ARGUS_HIP_ERR_UNSUPPORTED, "attention_gen_desc: declined, head_dim %d is not whole blocks of %u", a->head_dim, d->block_elems);
  if (d->block_elems == 32) {
    int named = -1;
    if (d->packing == 1 && d->bits == 4) named = d->scale_layout == 1 ? ARGUS_HIP_Q4_0 : ARGUS_HIP_Q4_1;
    else if (d->packing == 2 && d->scale_layout == 1) named = ARGUS_HIP_Q8_0;
    else if (d->packing == 3) named = ARGUS_HIP_Q2_0;
    if (named >= 0) {
      const int rc = attention_gen_impl(ctx, a, named, nullptr, 0);
      if (rc != ARGUS_HIP_ERR_UNSUPPORTED) return rc;  // shapes the block kernel refuses (wide GQA groups, unaligned rows) go on below
    }
  }
  return attention_gen_impl(ctx, a, kKvDesc, d, q + (d->scale_layout == 1 ? 2 : 4));
}
