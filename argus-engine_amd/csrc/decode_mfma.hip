// Split-KV flash-decode on the matrix cores: the F16-cache, no-soft-cap, contiguous-slot case of
// Backend::attention_gen (engine/src/backend.rs:284-295).
//
// The vector-ALU decode kernel spends ~8 FMAs per K/V element pair per query head; at 5.6 TB/s
// that keeps the VALUs ~60 % busy and is what limits it.  Here both products run as MFMAs whose
// operands are exactly what a 16-byte row load puts in a lane, so nothing goes through LDS and the
// VALUs only do the softmax:
//
//   S^T[token][head] = K . Q^T     v_mfma_f32_16x16x32_f16
//       A (m = token = lane%16, k-group = lane/16): 8 channels = one 16-byte chunk of the token's
//       K row.  Lane (j, r) loads chunk 4*kk + j of row r, so a wave's load covers 16 rows x 64 B.
//       B (n = head = lane%16): the same chunk of Q, pre-scaled, split into f16 hi + lo parts (two
//       MFMAs) so the logits keep f32-level accuracy.
//       D: lane (j, h) holds the logits of tokens 4j..4j+3 for head h.
//   O[head][channel] = P . V       v_mfma_f32_16x16x16_f16
//       A (m = head, k = 4j + e): P for tokens 4j..4j+3 -- the lane's own softmax results.
//       B (n = channel slot, k = 4j + e): lane group j loads rows 4j..4j+3 (one 16-byte piece
//       each); a 4x8 in-register transpose (v_pack/v_perm) turns them into one operand per channel.
//
// Up to 16 query heads per KV head share the pass.  Split partials and the combine pass are the
// ones of the vector-ALU kernel (decode_common.hpp).
#include "decode_common.hpp"

#include <algorithm>

namespace argus_decode {

namespace {

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));

template <int D>
struct MfmaShape {
  static constexpr int KK = D / 32;                 // QK k-steps (32 channels each)
  static constexpr int VC = (D >= 128) ? 8 : 4;     // halfs a lane loads per V row piece
  static constexpr int VSEG = D / (16 * VC);        // pieces per row per lane
  static constexpr int NACC = VC * VSEG;            // O accumulators (float4 each)
  static constexpr int MAXH = (D == 256) ? 8 : 16;  // query heads per KV head (bounds the merge LDS)
};

// dword 3 of a raw (untyped, unstrided) buffer descriptor on this target
constexpr int kBufferFlags = 0x00020000;

// Bounds-checked streaming (non-temporal) load of 8 or 16 bytes: byte offsets `voff` per lane,
// `soff` wave-uniform.
template <typename T>
__device__ __forceinline__ T buffer_load_stream(__amdgpu_buffer_rsrc_t rsrc, uint32_t voff, uint32_t soff);
template <>
__device__ __forceinline__ half8_t buffer_load_stream<half8_t>(__amdgpu_buffer_rsrc_t rsrc, uint32_t voff, uint32_t soff) {
  return __builtin_bit_cast(half8_t, __builtin_amdgcn_raw_buffer_load_b128(rsrc, voff, soff, 2));
}
template <>
__device__ __forceinline__ half4_t buffer_load_stream<half4_t>(__amdgpu_buffer_rsrc_t rsrc, uint32_t voff, uint32_t soff) {
  return __builtin_bit_cast(half4_t, __builtin_amdgcn_raw_buffer_load_b64(rsrc, voff, soff, 2));
}

template <int VC>
struct VPiece;
template <>
struct VPiece<8> { using type = half8_t; };
template <>
struct VPiece<4> { using type = half4_t; };

// Waves per workgroup, each taking every kWaves-th tile of the workgroup's chunk.  (Eight waves
// drawing tiles from a counter in LDS evened out the finish times of the workgroups but moved
// less data per microsecond: 27.4 us against 26.4 us on one 32K-token sequence.)
constexpr int kWaves = 4;

template <int D, int TW, bool SOFTCAP, bool INDEXED>
__global__ __launch_bounds__(64 * kWaves) void decode_mfma_kernel(const DecodeParams p) {
  using SH = MfmaShape<D>;
  constexpr int KK = SH::KK, VC = SH::VC, VSEG = SH::VSEG, NACC = SH::NACC;
  using vpiece_t = typename VPiece<VC>::type;
  constexpr int TILE = 16 * TW;  // tokens per wave iteration
  constexpr float kLn2 = 0.6931471805599453f, kLog2e = 1.4426950408889634f;
  const float inv_cap = SOFTCAP ? 1.0f / p.softcap : 0.0f;

  const int split = blockIdx.x, kvh = blockIdx.y, b = blockIdx.z;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int j = lane >> 4, r = lane & 15;
  const int G = p.group;

  const int t_begin = split * p.chunk;
  const int t_end = min(p.len, t_begin + p.chunk);

  const _Float16 *kb = (const _Float16 *)p.k + (int64_t)b * p.kv_bs + (int64_t)kvh * p.head_stride;
  const _Float16 *vb = (const _Float16 *)p.v + (int64_t)b * p.kv_bs + (int64_t)kvh * p.head_stride;

  // K/V rows are read through buffer descriptors that end at the chunk's last row: rows past it
  // come back as zeros without touching memory, so every iteration issues the same loads (the
  // compiler then waits for exactly the ones it needs) and a tile may be requested before it is
  // known to exist.  Offsets: a per-lane constant plus the wave-uniform first row of the tile.
  const int64_t rs = p.row_stride;
  const uint32_t slab_bytes = (uint32_t)((int64_t)(INDEXED ? p.slot_bound : p.kv_start + t_end) * rs * 2);
  const __amdgpu_buffer_rsrc_t k_rsrc = __builtin_amdgcn_make_buffer_rsrc((void *)kb, 0, slab_bytes, kBufferFlags);
  const __amdgpu_buffer_rsrc_t v_rsrc = __builtin_amdgcn_make_buffer_rsrc((void *)vb, 0, slab_bytes, kBufferFlags);
  const uint32_t k_lane = (uint32_t)(((int64_t)(p.kv_start + r) * rs + 8 * j) * 2);
  const uint32_t v_lane = (uint32_t)(((int64_t)(p.kv_start + 4 * j) * rs + VC * r) * 2);
  const uint32_t row_bytes = (uint32_t)(rs * 2);
  half8_t kr[TW][KK];
  vpiece_t vr[TW][VSEG][4];
  // With an index list (INDEXED: token t lives in slot kv_index[t]) the slots of the tile after next
  // are read from the list right behind the requests for the next tile, K slots behind the K
  // requests and V slots behind the V requests, so neither request waits on a load younger than
  // the data about to be used.  Tokens past the chunk re-read its last slot and are masked below.
  const int32_t *idx = INDEXED ? p.kv_index + (int64_t)b * p.index_bs : nullptr;
  const int last = t_end - 1;
  int k_slot[INDEXED ? TW : 1], v_slot[INDEXED ? 4 * TW : 1];
  auto load_idx_k = [&](int base) {
    if constexpr (INDEXED) {
#pragma unroll
      for (int tw = 0; tw < TW; ++tw) k_slot[tw] = idx[min(base + 16 * tw + r, last)];
    }
  };
  auto load_idx_v = [&](int base) {
    if constexpr (INDEXED) {
#pragma unroll
      for (int i = 0; i < 4 * TW; ++i) v_slot[i] = idx[min(base + 16 * (i >> 2) + 4 * j + (i & 3), last)];
    }
  };
  auto load_k = [&](int base) {  // TW tiles of 16 tokens starting at token `base`
    const uint32_t tile = (uint32_t)base * row_bytes;
#pragma unroll
    for (int tw = 0; tw < TW; ++tw)
#pragma unroll
      for (int kk = 0; kk < KK; ++kk) {
        if constexpr (INDEXED) kr[tw][kk] = buffer_load_stream<half8_t>(k_rsrc, __umul24((uint32_t)k_slot[tw], row_bytes) + 16 * j + 64 * kk, 0u);
        else kr[tw][kk] = buffer_load_stream<half8_t>(k_rsrc, k_lane + 16 * tw * row_bytes + 64 * kk, tile);
      }
  };
  auto load_v = [&](int base) {
    const uint32_t tile = (uint32_t)base * row_bytes;
#pragma unroll
    for (int tw = 0; tw < TW; ++tw)
#pragma unroll
      for (int e = 0; e < 4; ++e)
#pragma unroll
        for (int sg = 0; sg < VSEG; ++sg) {
          if constexpr (INDEXED)
            vr[tw][sg][e] = buffer_load_stream<vpiece_t>(v_rsrc, __umul24((uint32_t)v_slot[4 * tw + e], row_bytes) + 2 * VC * r + 32 * VC * sg, 0u);
          else
            vr[tw][sg][e] = buffer_load_stream<vpiece_t>(v_rsrc, v_lane + (16 * tw + e) * row_bytes + 32 * VC * sg, tile);
        }
  };
  // The first tile is requested before the query is prepared, so both arrive together.
  const int base0 = t_begin + __builtin_amdgcn_readfirstlane(wave) * TILE;
  load_idx_k(base0);
  load_idx_v(base0);
  load_k(base0);
  load_idx_k(base0 + kWaves * TILE);
  load_v(base0);
  load_idx_v(base0 + kWaves * TILE);
  __builtin_amdgcn_sched_barrier(0);  // keep these requests ahead of the query's

  // ---- Q operand: lane (j, h = r) holds chunk 4kk + j of head h, scaled to the log2 domain ------
  half8_t qh[KK], ql[KK];
  {
    const float c = p.scale * 1.4426950408889634f;
    const int h = kvh * G + min(r, G - 1);
    const float *qp = p.q + (int64_t)b * p.q_bs + (int64_t)h * D;
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
      float qv[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) qv[e] = qp[(4 * kk + j) * 8 + e];  // lanes past the group re-read its last head
      loaded8(qv);
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float x = (r < G) ? qv[e] * c : 0.0f;
        _Float16 hi, lo;
        split_f16(x, hi, lo);
        qh[kk][e] = hi;
        ql[kk][e] = lo;
      }
    }
  }

  // Dynamic LDS: the chunk's logits when they are staged (p.stage_scores: G rows of chunk + 4 floats),
  // then the merge area.
  extern __shared__ __attribute__((aligned(16))) float dyn_lds[];
  const int stage_row = p.chunk + 4;
  const int staged_heads = p.stage_scores ? p.group : 0;
  __shared__ __attribute__((aligned(16))) float logit_stage[kWaves][LogitSink<TW>::kStageFloats];
  // Lanes that park nothing write here: the sink's stage when the logits are staged (the sink is off
  // then), else the start of the dynamic area (the merge uses it after the loop only).
  static_assert(sizeof(logit_stage) >= 64 * kWaves * TW * 16, "spare slots of 16 TW bytes per lane");
  float *spare = p.stage_scores ? &logit_stage[0][0] : dyn_lds;
  const LogitSink<TW> sink(p, logit_stage[wave], b, kvh * G, G, lane, t_end);

  float4_t o_acc[NACC];
#pragma unroll
  for (int a = 0; a < NACC; ++a) o_acc[a] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
  float m_run = kNegInf, l_run = 0.0f;  // per (lane = head r); l is this lane group's partial sum
  int base_last = -(1 << 30);

  for (int base = base0; base < t_end; base += kWaves * TILE) {
    // ---- logits ---------------------------------------------------------------------------------
    float4_t s[TW];
#pragma unroll
    for (int tw = 0; tw < TW; ++tw) {
      s[tw] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
      for (int kk = 0; kk < KK; ++kk) {
        s[tw] = __builtin_amdgcn_mfma_f32_16x16x32_f16(kr[tw][kk], qh[kk], s[tw], 0, 0, 0);
        s[tw] = __builtin_amdgcn_mfma_f32_16x16x32_f16(kr[tw][kk], ql[kk], s[tw], 0, 0, 0);
      }
    }
    // The K registers are free again: request the wave's next tile (past the chunk: zeros, no traffic).
    load_k(base + kWaves * TILE);
    load_idx_k(base + 2 * kWaves * TILE);
    const bool full = base + TILE <= t_end;
    float mt = kNegInf;
#pragma unroll
    for (int tw = 0; tw < TW; ++tw)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float sv = s[tw][i];
        if constexpr (SOFTCAP) {
          // cap * tanh(logit / cap) on the natural-unit logit (flash_attn_f32_f16.cl:563-565), back to log2 units
          const float capped = softcap_tanh(sv * kLn2, p.softcap, inv_cap) * kLog2e;
          sv = (sv != sv) ? kNegInf : capped;
        }
        sv = fmaxf(sv, kNegInf);  // NaN logit counts as -inf (common.rs:555-560)
        if (!full && base + 16 * tw + 4 * j + i >= t_end) sv = kNegInf;
        s[tw][i] = sv;
        mt = fmaxf(mt, sv);
      }
    // Staged or not, the iteration issues the sink's one store (dropped when it has nothing to write):
    // a store on one side of a branch only would make the compiler's wait counts inexact.
    stage_logits<TW>(dyn_lds, stage_row, r, j, staged_heads, base - t_begin, s, spare);
    sink.store(s, base);
    base_last = base;

    // ---- online softmax: the running max of a head is shared by the four lane groups -----------
    mt = rows_allreduce_max(mt);
    const float m_new = fmaxf(m_run, mt);
    const float m_ref = (m_new == kNegInf) ? 0.0f : m_new;
    const float alpha = __builtin_amdgcn_exp2f(m_run - m_ref);
    m_run = m_new;
    half4_t pa[TW];
    float lsum = 0.0f;
#pragma unroll
    for (int tw = 0; tw < TW; ++tw) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        // The row sum takes the unrounded weight: it also normalises the emitted scores, and over a
        // few dozen tokens the f16 roundings of the weights do not average out (1.1e-4 at L = 65).
        const float w = __builtin_amdgcn_exp2f(s[tw][i] - m_ref);
        lsum += w;
        pa[tw][i] = (_Float16)w;
      }
    }
    l_run = l_run * alpha + lsum;
    if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0) {
      // O accumulator register i of lane group j belongs to head 4j + i: fetch that head's factor.
      float al[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) al[i] = __shfl(alpha, 4 * j + i, 64);
#pragma unroll
      for (int a = 0; a < NACC; ++a)
#pragma unroll
        for (int i = 0; i < 4; ++i) o_acc[a][i] *= al[i];
    }

    // ---- O += P . V -----------------------------------------------------------------------------
#pragma unroll
    for (int tw = 0; tw < TW; ++tw)
#pragma unroll
      for (int sg = 0; sg < VSEG; ++sg)
#pragma unroll
        for (int c = 0; c < VC; ++c) {
          const half4_t bv = {vr[tw][sg][0][c], vr[tw][sg][1][c], vr[tw][sg][2][c], vr[tw][sg][3][c]};
          o_acc[sg * VC + c] = __builtin_amdgcn_mfma_f32_16x16x16f16(pa[tw], bv, o_acc[sg * VC + c], 0, 0, 0);
        }
    load_v(base + kWaves * TILE);
    load_idx_v(base + 2 * kWaves * TILE);
  }
  if (p.stage_scores) {
    flush_staged_logits(p, dyn_lds, stage_row, b, kvh * G, G, t_begin, t_end);
  } else {
    sink.store_tail(base_last);
    __syncthreads();  // the other waves' spare slots lie in the merge area
  }

  // ---- merge: lane groups (row sum), then the waves through LDS ---------------------------------
  l_run += __shfl_xor(l_run, 16, 64);
  l_run += __shfl_xor(l_run, 32, 64);
  float (*lds_m)[16] = (float (*)[16])dyn_lds;
  float (*lds_l)[16] = lds_m + kWaves;
  float (*lds_acc)[SH::MAXH][D + 4] = (float (*)[SH::MAXH][D + 4])(dyn_lds + 2 * kWaves * 16);
  if (j == 0) {
    lds_m[wave][r] = m_run;
    lds_l[wave][r] = l_run;
  }
#pragma unroll
  for (int sg = 0; sg < VSEG; ++sg)
#pragma unroll
    for (int c = 0; c < VC; ++c)
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (4 * j + i < SH::MAXH) lds_acc[wave][4 * j + i][16 * VC * sg + VC * r + c] = o_acc[sg * VC + c][i];
  __syncthreads();

  for (int idx = threadIdx.x; idx < G * D; idx += 64 * kWaves) {
    const int g = idx / D, c = idx % D;
    const int h = kvh * G + g;
    float mm = lds_m[0][g];
#pragma unroll
    for (int w = 1; w < kWaves; ++w) mm = fmaxf(mm, lds_m[w][g]);
    const float m_ref = (mm == kNegInf) ? 0.0f : mm;
    float o = 0.0f, ll = 0.0f;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) {
      const float f = __builtin_amdgcn_exp2f(lds_m[w][g] - m_ref);
      o += lds_acc[w][g][c] * f;
      ll += lds_l[w][g] * f;
    }
    if (p.direct) {
      // One split and no scores: the row is finished here and no combine pass follows.  A row
      // without any finite logit is left to the fallback below.
      if (ll > 0.0f && ll < __builtin_huge_valf()) p.out[(int64_t)b * p.out_bs + (int64_t)h * D + c] = o / ll;
      continue;
    }
    // Partials are handed to the combine pass in natural-log units.
    const int64_t pidx = ((int64_t)b * p.n_heads_q + h) * p.nsplit + split;
    p.ws_o[pidx * D + c] = o;
    if (c == 0) {
      p.ws_ml[pidx * 2 + 0] = mm * kLn2;
      p.ws_ml[pidx * 2 + 1] = ll;
    }
  }
  if (p.direct) {
    for (int g = 0; g < G; ++g) {
      float mm = lds_m[0][g];
#pragma unroll
      for (int w = 1; w < kWaves; ++w) mm = fmaxf(mm, lds_m[w][g]);
      const float m_ref = (mm == kNegInf) ? 0.0f : mm;
      float ll = 0.0f;
#pragma unroll
      for (int w = 0; w < kWaves; ++w) ll += lds_l[w][g] * __builtin_amdgcn_exp2f(lds_m[w][g] - m_ref);
      if (!(ll > 0.0f && ll < __builtin_huge_valf())) uniform_fallback<_Float16>(p, b, kvh * G + g, D);  // uniform per workgroup
    }
  }
}

template <int D>
int launch_mfma(argus_hip_ctx *ctx, DecodeParams &p, int batch, hipStream_t stream) {
  constexpr int TW = (D <= 128) ? 2 : 1;
  constexpr int tile_rows = kWaves * 16 * TW;  // one tile per wave
  const int pairs = batch * p.n_heads_kv;
  // With scores the chunks are kept short enough for a workgroup's logits to wait in LDS until its
  // token loop is over (kStageBytes; two workgroups per CU still fit beside the 9 KB of static LDS).
  // 66 KB and not 64: a group of four heads then stages chunks of 4096 tokens (4 x 4100 floats), so a
  // 32K-token row is 8 chunks and 16 sequences x 8 KV heads fill exactly two resident rounds; at
  // 64 KB the same row took 9 chunks, i.e. 2.25 rounds, and the thin third round cost 30 % of the
  // launch.  The resident round is counted at the LDS size the launch may reach.
  constexpr int kStageBytes = 66 * 1024;
  constexpr size_t merge_bytes = (2 * kWaves * 16 + kWaves * MfmaShape<D>::MAXH * (D + 4)) * sizeof(float);
  const int max_chunk = staged_chunk_limit(ctx, p, kStageBytes, tile_rows);
  const int wgs_per_cu = argus_wgs_per_cu(ctx, decode_mfma_kernel<D, TW, false, false>, 64 * kWaves,
                                          max_chunk > 0 ? (size_t)kStageBytes : merge_bytes);
  choose_splits(p, pairs, tile_rows, (int64_t)ctx->compute_units * wgs_per_cu, max_chunk, p.scores ? 0.0f : 1.5f);
  p.direct = (p.nsplit == 1 && !p.scores) ? 1 : 0;  // the split pass writes `out` itself: one launch
  p.stage_scores = p.scores && p.chunk <= max_chunk;
  const size_t lds_bytes = std::max(merge_bytes, p.stage_scores ? (size_t)p.group * (p.chunk + 4) * sizeof(float) : (size_t)0);
  const bool cap = p.softcap > 0.0f, indexed = p.kv_index != nullptr;
  auto kern = cap ? (indexed ? decode_mfma_kernel<D, TW, true, true> : decode_mfma_kernel<D, TW, true, false>)
                  : (indexed ? decode_mfma_kernel<D, TW, false, true> : decode_mfma_kernel<D, TW, false, false>);
  ARGUS_HIP_CHECK(ctx, argus_raise_lds_limit(ctx, kern, kStageBytes + 1024));
  if (!p.direct) {
    const int rc = reserve_partials(ctx, p, batch, D);
    if (rc != ARGUS_HIP_OK) return rc;
  }
  ctx->plan = argus_hip_decode_plan{p.nsplit, p.chunk, wgs_per_cu, (int32_t)lds_bytes, p.direct ? 1 : 2, 1, p.stage_scores};
  KernelTimer timer(ctx, stream);
  hipLaunchKernelGGL(kern, dim3(p.nsplit, p.n_heads_kv, batch), dim3(64 * kWaves), lds_bytes, stream, p);
  timer.mark();
  if (p.direct) return hipGetLastError() == hipSuccess ? ARGUS_HIP_OK : argus_fail(ctx, ARGUS_HIP_ERR_RUNTIME, "decode launch failed");
  ARGUS_HIP_CHECK(ctx, hipGetLastError());
  hipLaunchKernelGGL((decode_combine_kernel<UniformFallback<_Float16>, D>), combine_grid(p, batch), dim3(256), 0, stream, p);
  ARGUS_HIP_CHECK(ctx, hipGetLastError());
  return ARGUS_HIP_OK;
}

}  // namespace

bool decode_mfma_supported(const DecodeParams &p, int D, int kv_dtype, int batch) {
  if (kv_dtype != ARGUS_HIP_F16 || p.len < 64) return false;
  // rows are addressed with 32-bit byte offsets from the head's first row, a few tiles past the end;
  // an index list may name any slot of the cache (slot x row bytes is a 24-bit multiply)
  const int64_t rows = p.kv_index ? p.slot_bound : (int64_t)p.kv_start + p.len;
  if ((rows + 1024) * p.row_stride * 2 > 0x7fffffffll) return false;
  if (p.kv_index && (rows >= (1 << 24) || p.row_stride * 2 >= (1 << 24))) return false;
  if (!score_rows_addressable(p)) return false;
  if (D == 64 || D == 128) return p.group <= 16;
  // head_dim 256: one 64-row tile per workgroup costs more set-up (Q split over 256 channels) than it
  // saves on short calls; measured against the vector-ALU kernel it pays for long rows with wider
  // groups (Hq8/Hkv4, L 2048: 30 us vs 17 us; L 32768: equal) and, with two to three heads per KV
  // head, once the call attends enough rows in total (Hq8/Hkv4, L 2048, scores and soft cap: 17.0 vs
  // 14.9 us at 8 sequences, 80 vs 101 us at 64; the lines cross near 13 sequences).
  if (D != 256 || p.group > 8) return false;
  if (p.group >= 4) return p.len >= 8192;
  return (int64_t)batch * p.n_heads_kv * p.len >= 128 * 1024;
}

int launch_decode_mfma(argus_hip_ctx *ctx, DecodeParams &p, int D, int batch, hipStream_t stream) {
  switch (D) {
    case 64: return launch_mfma<64>(ctx, p, batch, stream);
    case 128: return launch_mfma<128>(ctx, p, batch, stream);
    default: return launch_mfma<256>(ctx, p, batch, stream);
  }
}

}  // namespace argus_decode
