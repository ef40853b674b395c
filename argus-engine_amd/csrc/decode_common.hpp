// Pieces shared by the split-KV decode kernels (F16/F32 cache and KIVI-quantised cache):
// launch parameters, the soft-cap, the uniform-weights fallback and the split-combine pass.
#pragma once

#include "argus_hip_internal.hpp"

#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <type_traits>

namespace argus_decode {

struct DecodeParams {
  const float *q;
  const void *k;
  const void *v;
  float *out;
  float *scores;
  // When set, `scores` keeps the logits and the combine pass writes each row's (max, sum) here
  // instead of rewriting the row as probabilities: [batch, Hq, 2], batch stride stats_bs.
  float *score_stats;
  const int32_t *kv_index;
  float *ws_ml;  // [batch, Hq, nsplit, 2]
  float *ws_o;   // [batch, Hq, nsplit, D]
  int32_t n_heads_q, n_heads_kv, group;  // group = Hq / Hkv
  int32_t len, kv_start, chunk, nsplit;
  int32_t score_stride;
  int64_t row_stride;   // elements between consecutive token rows of one KV head
  int64_t head_stride;  // elements between KV heads
  int64_t q_bs, out_bs, kv_bs, score_bs, index_bs, stats_bs;
  float scale, softcap;
  int32_t direct;  // nsplit == 1 and no scores: first pass writes `out` itself
  int32_t slot_bound;  // slots an index list may name (the cache capacity)
  int32_t head_chunks; // vector-ALU kernel: workgroups per KV head (GQA groups wider than its head tile)
  int32_t stage_scores;  // matrix-core kernels: the chunk's logits wait in LDS and are written after the token loop
  // Descriptor-driven rows (vector-ALU kernel only): KVLayoutDesc of the cache and its block size in bytes.
  int32_t desc_block_elems, desc_bits, desc_scale_layout, desc_packing, desc_block_bytes;
};

// Tag type of a cache whose rows are blocks described by a KVLayoutDesc (any PerBlockF16[WithMin] x
// Nibble / Byte / Quad descriptor, engine/src/format/dtype_layout.rs:102-166).
struct DescRow {};

// Elements w0 .. w0+7 (w0 a multiple of 8) of the block at `blk`, decoded like
// unpack_block_via_descriptor: nibble packing keeps element i < n/2 in the low nibble of byte i and
// element n/2 + i in the high nibble; signed with zero point 2^(bits-1) when the block has no
// minimum, else code * scale + min; byte packing is a signed i8; quad packing holds elements
// 4i .. 4i+3 of byte i at bit offsets 0/2/4/6.  Blocks are only 2-byte aligned.
__device__ __forceinline__ void desc_decode8(const DecodeParams &p, const uint8_t *blk, int w0, float (&out)[8]) {
  const float scale = (float)*(const _Float16 *)blk;
  const bool has_min = p.desc_scale_layout == 2;
  const float mn = has_min ? (float)*(const _Float16 *)(blk + 2) : 0.0f;
  const uint8_t *q = blk + (has_min ? 4 : 2);
  if (p.desc_packing == 1) {
    const int half = p.desc_block_elems / 2, zp = 1 << (p.desc_bits - 1);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int i = w0 + e;
      const int b = (int)q[i < half ? i : i - half];
      const int code = i < half ? (b & 0x0f) : (b >> 4);
      out[e] = has_min ? __fadd_rn(__fmul_rn((float)code, scale), mn) : __fmul_rn((float)(code - zp), scale);
    }
  } else if (p.desc_packing == 2) {
#pragma unroll
    for (int e = 0; e < 8; ++e) out[e] = __fmul_rn((float)(int)(int8_t)q[w0 + e], scale);
  } else {
    const uint32_t w = (uint32_t)q[w0 / 4] | ((uint32_t)q[w0 / 4 + 1] << 8);
#pragma unroll
    for (int e = 0; e < 8; ++e) out[e] = __fadd_rn(__fmul_rn((float)((w >> (2 * e)) & 3u), scale), mn);
  }
}
// Byte offset of the block that holds element `elem` (a multiple of the block size apart from the
// position inside the block) of a cache addressed in elements.
__device__ __forceinline__ int64_t desc_block_offset(const DecodeParams &p, int64_t elem) {
  return elem / p.desc_block_elems * p.desc_block_bytes;
}

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
      const int64_t slot = idx ? (int64_t)min((uint32_t)idx[t], (uint32_t)(p.slot_bound - 1)) : (p.kv_start + t);
      acc += u * (float)vb[slot * p.row_stride + c];
    }
    p.out[(int64_t)b * p.out_bs + (int64_t)h * D + c] = acc;
  }
  if (p.scores) {
    float *srow = p.scores + (int64_t)b * p.score_bs + (int64_t)h * p.score_stride;
    // (logits + statistics form: exp(0 - 0) / len is the same uniform weight)
    for (int t = threadIdx.x; t < p.len; t += blockDim.x) srow[t] = p.score_stats ? 0.0f : u;
    if (p.score_stats && threadIdx.x == 0) {
      float *st = p.score_stats + (int64_t)b * p.stats_bs + (int64_t)h * 2;
      st[0] = 0.0f;
      st[1] = (float)p.len;
    }
  }
}

template <>
__device__ inline void uniform_fallback<DescRow>(const DecodeParams &p, int b, int h, int D) {
  const int kvh = h / p.group;
  const uint8_t *vb = (const uint8_t *)p.v;
  const int32_t *idx = p.kv_index ? p.kv_index + (int64_t)b * p.index_bs : nullptr;
  const float u = 1.0f / (float)p.len;
  for (int c8 = threadIdx.x; c8 < D / 8; c8 += blockDim.x) {
    float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    for (int t = 0; t < p.len; ++t) {
      const int64_t slot = idx ? (int64_t)min((uint32_t)idx[t], (uint32_t)(p.slot_bound - 1)) : (p.kv_start + t);
      const int64_t elem = (int64_t)b * p.kv_bs + (int64_t)kvh * p.head_stride + slot * p.row_stride + 8 * c8;
      float v[8];
      desc_decode8(p, vb + desc_block_offset(p, elem), (int)(elem % p.desc_block_elems), v);
      for (int e = 0; e < 8; ++e) acc[e] += u * v[e];
    }
    for (int e = 0; e < 8; ++e) p.out[(int64_t)b * p.out_bs + (int64_t)h * D + 8 * c8 + e] = acc[e];
  }
  if (p.scores) {
    float *srow = p.scores + (int64_t)b * p.score_bs + (int64_t)h * p.score_stride;
    // (logits + statistics form: exp(0 - 0) / len is the same uniform weight)
    for (int t = threadIdx.x; t < p.len; t += blockDim.x) srow[t] = p.score_stats ? 0.0f : u;
    if (p.score_stats && threadIdx.x == 0) {
      float *st = p.score_stats + (int64_t)b * p.stats_bs + (int64_t)h * 2;
      st[0] = 0.0f;
      st[1] = (float)p.len;
    }
  }
}

// Fallback policies of the combine pass when a row has no finite logit.
template <typename KV_T>
struct UniformFallback {
  // Scalar reference behaviour (common.rs:561-577): uniform weights.
  static constexpr bool kHandlesRow = true;  // run() writes the whole output and score row
  static __device__ bool run(const DecodeParams &p, int b, int h, int D) {
    uniform_fallback<KV_T>(p, b, h, D);
    return true;
  }
};
struct NoFallback {
  // The reference KIVI kernels have no guard (kivi_attn.cu:252-390): NaN propagates.
  static constexpr bool kHandlesRow = false;
  static __device__ bool run(const DecodeParams &, int, int, int) { return false; }
};

// Second pass: log-sum-exp merge of the splits of one (sequence, Q head); optional in-place
// logits -> probabilities rewrite of the score row.  The 256 threads are arranged as
// (split group) x (float4 column) so the loop over splits is short and the loads are wide.
// A long score row is shared between gridDim.z workgroups: each merges the (m, l) pairs for
// itself (a few hundred bytes), the first also writes the output row, and every one rewrites its
// slice of the scores (one workgroup per 32K-token row took 40 us).
constexpr int kMaxSplits = 128;

template <typename FALLBACK, int D>
__global__ __launch_bounds__(256) void decode_combine_kernel(const DecodeParams p) {
  constexpr int CQ = D / 4;                // float4 columns per row
  constexpr int NSG = 256 / CQ;            // split groups
  constexpr int PER = kMaxSplits / NSG;    // splits per thread at most
  const int h = blockIdx.x, b = blockIdx.y;
  const bool first = blockIdx.z == 0;  // the workgroup that also merges the output row
  const int64_t pbase = ((int64_t)b * p.n_heads_q + h) * p.nsplit;
  const int cq = threadIdx.x % CQ, sg = threadIdx.x / CQ;
  __shared__ float sh_w[kMaxSplits];
  __shared__ float sh_m, sh_l;
  __shared__ float4_t sh_o[NSG][CQ];
  // The pass is one memory round trip long if nothing waits on anything else, so the partial
  // outputs are requested before the (m, l) pairs that weight them.  Slots past the last split
  // re-read it and get weight zero.
  const int last = p.nsplit - 1;
  // The logits of the workgroup's slice of the score row are requested first of all (the usual
  // slice is 4096 tokens, kAhead per thread), so the rewrite does not start a second round trip
  // once the row's maximum and sum are known.
  constexpr int kAhead = 16;
  const bool rewrite = p.scores && !p.score_stats;  // else the row keeps its logits and only (max, sum) are written
  float *srow = p.scores ? p.scores + (int64_t)b * p.score_bs + (int64_t)h * p.score_stride : nullptr;
  const int slice = ((p.len + (int)gridDim.z - 1) / (int)gridDim.z + 255) / 256 * 256;
  const int t_end = min(p.len, ((int)blockIdx.z + 1) * slice);
  const int t0 = (int)blockIdx.z * slice + (int)threadIdx.x;
  // Rows that start on a 16-byte boundary are read and written as float4: thread x then owns the
  // tokens 4 (x + 256 k) .. + 3 of the slice's first 4096 instead of x + 256 k (k < kAhead).
  const bool vec = rewrite && (((uintptr_t)srow) & 15) == 0;
  const int s0 = (int)blockIdx.z * slice;
  float logit[kAhead];
  if (rewrite) {
    if (vec) {
#pragma unroll
      for (int k = 0; k < kAhead / 4; ++k) {
        const int tv = s0 + 4 * ((int)threadIdx.x + 256 * k);
        if (tv + 3 < p.len) {
          const float4_t v = __builtin_nontemporal_load((const float4_t *)(srow + tv));
#pragma unroll
          for (int e = 0; e < 4; ++e) logit[4 * k + e] = v[e];
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e) logit[4 * k + e] = __builtin_nontemporal_load(srow + min(tv + e, p.len - 1));
        }
      }
    } else {
#pragma unroll
      for (int k = 0; k < kAhead; ++k) logit[k] = __builtin_nontemporal_load(srow + min(t0 + 256 * k, p.len - 1));
    }
  }
  float4_t part[PER];
  if (first) {
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      if (i * NSG > last) break;  // uniform
      part[i] = *(const float4_t *)(p.ws_o + (pbase + min(sg + i * NSG, last)) * D + 4 * cq);
    }
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
    if (!first && FALLBACK::kHandlesRow) return;  // the first workgroup writes the whole row
    if (first && FALLBACK::run(p, b, h, D)) return;
  }
  const float inv = 1.0f / ll;  // non-finite when the fallback declined: NaN propagates
  if (first && p.score_stats && threadIdx.x == 0) {
    float *st = p.score_stats + (int64_t)b * p.stats_bs + (int64_t)h * 2;
    st[0] = mm;
    st[1] = ll;
  }
  if (first) {
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
  }
  if (rewrite) {
    if (vec) {
#pragma unroll
      for (int k = 0; k < kAhead / 4; ++k) {
        const int tv = s0 + 4 * ((int)threadIdx.x + 256 * k);
        float4_t v;
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = __expf(logit[4 * k + e] - mm) * inv;
        if (tv + 3 < t_end) {
          __builtin_nontemporal_store(v, (float4_t *)(srow + tv));
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (tv + e < t_end) __builtin_nontemporal_store(v[e], srow + tv + e);
        }
      }
    } else {
#pragma unroll
      for (int k = 0; k < kAhead; ++k) {
        const int t = t0 + 256 * k;
        if (t < t_end) __builtin_nontemporal_store(__expf(logit[k] - mm) * inv, srow + t);
      }
    }
    for (int t = t0 + 256 * kAhead; t < t_end; t += 256)
      __builtin_nontemporal_store(__expf(__builtin_nontemporal_load(srow + t) - mm) * inv, srow + t);
  }
}

// Where the matrix-core kernels put their logits (natural units; the combine pass rewrites them as
// probabilities).  Out of the MFMA a lane (j, r) holds tokens 4j..4j+3 of head r for each 16-token
// tile, so a store from those registers hands the memory system sixteen 16-byte pieces of sixteen
// different lines per instruction.  The wave turns its TW tiles round in LDS instead: eight
// consecutive lanes take one head's 16 TW tokens, and one instruction writes whole lines of eight
// heads.
// The stores go through a buffer descriptor over the score rows of the KV head's group: heads past
// the group, token groups that reach past the chunk and a call without `scores` (zero records)
// carry an offset outside it and the hardware drops them.  Every iteration of the token loop then
// issues the same store with no branch around it, which keeps the compiler's counts of outstanding
// memory operations exact (with a store on one side of a branch it assumes none, and the wait for a
// V tile comes to include the first requests of the K tile just asked for).  A chunk ends inside a
// lane's token group only at the end of the row; that group is written after the loop (store_tail).
// Groups of more than 8 heads take a second store under a branch.  Rows of at most 2 GiB per group:
// score_rows_addressable().
// What the stores cost is set by the bytes written, not by their form: 32 heads x 32K tokens x 16
// sequences (67 MB of logits beside 2.1 GB of K and V) take the F16 kernel from 302 to 426 us with
// per-lane stores under a branch, with branch-free stores and with the whole-line stores below
// alike; the staging alone is free (304 us with the store left out), a quarter of the stores costs
// 355 us, the same stores confined to 4 KB per row (no DRAM writes) 393 us, and the fetch counter
// shows no extra reads.  Part of it is the wave's own loads waiting behind its stores (loads and
// stores of a wave retire in order): the F16 kernel therefore keeps a chunk's logits in LDS and
// writes them when its token loop is over, where the chunk fits (DecodeParams::stage_scores:
// 390 us), and uses this sink where it does not.  The rest is writes mixed into a saturated read
// stream: 64 MB filled by another kernel meanwhile cost the plain launch 40 us as well.
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
template <int TW>
struct LogitSink {
  static_assert(TW == 1 || TW == 2, "one or two 16-token tiles per wave iteration");
  static constexpr int T = 16 * TW, ROW = T + 4, VEC = 2 * TW;  // in floats; ROW keeps 16-byte alignment
  static constexpr int kStageFloats = 16 * ROW;                 // per wave
  static constexpr uint32_t kDropped = 0x80000000u;
  static constexpr float kLn2 = 0.6931471805599453f;
  using vec_t = typename std::conditional<TW == 2, u32x4_t, u32x2_t>::type;

  __amdgpu_buffer_rsrc_t rsrc;
  uint32_t off[2];  // byte offset of the lane's first token in its row, for heads 0..7 and 8..15
  float *wr;        // where lane (j, r) puts a tile's four logits
  const float *rd;  // the lane's VEC tokens of head lane / 8
  int tok, t_end;
  bool on, wide;

  __device__ __forceinline__ LogitSink(const DecodeParams &p, float *stage, int b, int first_head, int heads, int lane, int t_end_)
      : t_end(t_end_) {
    on = p.scores != nullptr && !p.stage_scores;  // staged logits are written after the loop: every store here is dropped
    const uint32_t bytes = on ? (uint32_t)((((int64_t)heads - 1) * p.score_stride + t_end_) * 4) : 0u;
    void *rows = on ? (void *)(p.scores + (int64_t)b * p.score_bs + (int64_t)first_head * p.score_stride) : nullptr;
    rsrc = __builtin_amdgcn_make_buffer_rsrc(rows, 0, bytes, 0x00020000);
    wide = heads > 8;
    tok = VEC * (lane & 7);
#pragma unroll
    for (int n = 0; n < 2; ++n) {
      const int row = 8 * n + (lane >> 3);
      off[n] = (row < heads) ? (uint32_t)(((int64_t)row * p.score_stride + tok) * 4) : kDropped;
    }
    wr = stage + (lane & 15) * ROW + 4 * (lane >> 4);
    rd = stage + (lane >> 3) * ROW + tok;
  }

  static __device__ __forceinline__ void wave_fence() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  }
  __device__ __forceinline__ void emit(vec_t v, int n, int base) const {
    const uint32_t o = (base + tok + VEC <= t_end) ? off[n] + 4u * (uint32_t)base : kDropped;
    // non-temporal (aux bit 1): the logits are read back once by the combine pass and never by this kernel
    if constexpr (TW == 2) __builtin_amdgcn_raw_buffer_store_b128(v, rsrc, o, 0u, 2);
    else __builtin_amdgcn_raw_buffer_store_b64(v, rsrc, o, 0u, 2);
  }

  // `s`: the lane's logits of the TW tiles starting at token `base`, in log2 units.
  __device__ __forceinline__ void store(const float4_t (&s)[TW], int base) const {
    vec_t v0 = {}, v1 = {};
    if (on) {  // uniform; LDS traffic only
      wave_fence();  // the reads of the previous iteration are done
#pragma unroll
      for (int tw = 0; tw < TW; ++tw) *(float4_t *)(wr + 16 * tw) = s[tw] * kLn2;
      wave_fence();
      v0 = *(const vec_t *)rd;
      if (wide) v1 = *(const vec_t *)(rd + 8 * ROW);
    }
    emit(v0, 0, base);
    if (wide) emit(v1, 1, base);
  }
  // The token group that the end of the row cuts, if any.  `base`: the wave's last call of store(),
  // whose logits the stage still holds.
  __device__ __forceinline__ void store_tail(int base) const {
    if (!on || (t_end % VEC) == 0 || base + T <= t_end) return;
    for (int n = 0; n < (wide ? 2 : 1); ++n)
#pragma unroll
      for (int e = 0; e < VEC - 1; ++e) {
        const int t = base + tok + e;
        const bool cut = t < t_end && base + tok + VEC > t_end;
        const float x = rd[n * 8 * ROW + e];
        __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(uint32_t, x), rsrc, cut ? off[n] + 4u * (uint32_t)(base + e) : kDropped, 0u, 2);
      }
  }
};
// Staged score emission (DecodeParams::stage_scores): lane (j, r) parks a tile's four logits of head r
// in the workgroup's dynamic LDS, rows of `stage_row` floats per head, and the workgroup writes the
// chunk's rows once its token loop is over, when none of its loads is in flight any more.
// Branch-free on purpose (a branch here cuts the token loop's one basic block in two, and the
// block-cache kernels then lose 10 % of their rate): lanes with nothing to park (heads past the
// group, or staging off: `staged_heads` 0) write to a 16 TW-byte slot of their own in `spare`, an
// area of 64 TW bytes per wave lane that nothing else uses during the loop.
template <int TW>
__device__ __forceinline__ void stage_logits(float *stage, int stage_row, int r, int j, int staged_heads, int tok, const float4_t (&s)[TW],
                                             float *spare) {
  constexpr float kLn2 = 0.6931471805599453f;
  const bool parks = r < staged_heads;
  float *dst = parks ? stage + r * stage_row + tok + 4 * j : spare + 4 * TW * (int)threadIdx.x;
  const int step = parks ? 16 : 4;
#pragma unroll
  for (int tw = 0; tw < TW; ++tw) *(float4_t *)(dst + step * tw) = s[tw] * kLn2;
}
// The stores are non-temporal: 67 MB of logits written with default stores beside 2.1 GB of K and V
// reads took the F16 kernel from 304 to 372 us (32 heads x 32K tokens x 16 sequences), written
// non-temporally 338 us; the combine pass reads them back once, non-temporally too.
__device__ __forceinline__ void flush_staged_logits(const DecodeParams &p, const float *stage, int stage_row, int b, int first_head,
                                                    int heads, int t_begin, int t_end) {
  __syncthreads();
  const int n = t_end - t_begin;
  for (int g = 0; g < heads; ++g) {
    float *srow = p.scores + (int64_t)b * p.score_bs + (int64_t)(first_head + g) * p.score_stride + t_begin;
    const float *lrow = stage + g * stage_row;
    const int n4 = ((((uintptr_t)srow) & 15) == 0) ? n / 4 : 0;  // 16-byte stores where the row allows them
    for (int t = threadIdx.x; t < n4; t += blockDim.x) __builtin_nontemporal_store(*(const float4_t *)(lrow + 4 * t), (float4_t *)(srow + 4 * t));
    for (int t = 4 * n4 + threadIdx.x; t < n; t += blockDim.x) srow[t] = lrow[t];
  }
  __syncthreads();  // the caller reuses the area
}
// Longest chunk whose logits fit `stage_bytes` of LDS (0 without scores), for choose_splits().
// ARGUS_HIP_SCORES=direct (read when the context is created) keeps the stores in the token loop, the
// path of chunks too long to stage: for A/B measurements and for tests of that path at small sizes.
inline int staged_chunk_limit(const argus_hip_ctx *ctx, const DecodeParams &p, int stage_bytes, int tile_rows) {
  if (!p.scores || ctx->env.scores_direct) return 0;
  return (stage_bytes / 4 / p.group - 4) / tile_rows * tile_rows;
}
// Places the split partials of a launch (p.nsplit set) in the context workspace.
inline int reserve_partials(argus_hip_ctx *ctx, DecodeParams &p, int batch, int D) {
  const size_t n_part = (size_t)batch * p.n_heads_q * p.nsplit;
  const size_t ml_bytes = (n_part * 2 * sizeof(float) + 255) / 256 * 256;
  const int rc = argus_ws_reserve(ctx, ml_bytes + n_part * D * sizeof(float));
  if (rc != ARGUS_HIP_OK) return rc;
  p.ws_ml = argus_ws(ctx);
  p.ws_o = (float *)((char *)argus_ws(ctx) + ml_bytes);
  return ARGUS_HIP_OK;
}
inline bool score_rows_addressable(const DecodeParams &p) {
  return !p.scores || (p.score_stride >= p.len && ((int64_t)p.group * p.score_stride + 1024) * 4 <= 0x7fffffffll);
}

// Grid of the combine pass: one workgroup per (head, sequence), more along z for long score rows.
inline dim3 combine_grid(const DecodeParams &p, int batch) {
  const int z = (p.scores && !p.score_stats) ? std::max(1, std::min(64, p.len / 4096)) : 1;
  return dim3((unsigned)p.n_heads_q, (unsigned)batch, (unsigned)z);
}

// Split count of the matrix-core kernels.  The grid is sized against the number of workgroups the
// device holds at once (`slots`): when the splits fill it in one round every workgroup starts
// together and streams an equal share, each wave requesting its next tile while it works on the
// current one; a partial extra round runs thinly occupied (one 32K-token sequence: 2 rounds of
// 2-tile waves were 10 % slower than 1 round of 4-tile waves).  Cost model, in units of one tile
// step with the device full: rounds x (tile steps per workgroup + 0.75 for set-up, merge and
// partial write-out).  Sets p.nsplit and p.chunk (a multiple of tile_rows).
// `max_chunk` > 0: no chunk longer than that many tokens, when the split limit allows it.
// `second_launch`: what the combine pass costs a plan with more than one split, in the same unit,
// for launchers whose single-split plan needs no combine (it writes the output itself).  A lone
// workgroup walks its tile steps one memory round trip after the other, so the single launch only
// pays for rows of up to two tile steps: a 32-layer decode loop replayed as a HIP graph, every layer
// with a cache of its own, takes 250 against 271 us per token at 256 tokens of context with one
// launch per layer, but 373 against 285 us at 512 tokens (four steps).
inline void choose_splits(DecodeParams &p, int pairs, int tile_rows, int64_t slots, int max_chunk = 0, float second_launch = 0.0f) {
  const int max_splits = std::min((p.len + tile_rows - 1) / tile_rows, kMaxSplits);
  int nsplit = 1, chunk = (p.len + tile_rows - 1) / tile_rows * tile_rows;
  float best = 3.0e38f;
  for (int n = 1; n <= max_splits; ++n) {
    const int c = ((p.len + n - 1) / n + tile_rows - 1) / tile_rows * tile_rows;
    if (max_chunk > 0 && c > max_chunk && n < max_splits) continue;
    const int ns = (p.len + c - 1) / c;
    const int64_t rounds = ((int64_t)pairs * ns + slots - 1) / slots;
    const float cost = (float)rounds * ((float)(c / tile_rows) + 0.75f) + (ns > 1 ? second_launch : 0.0f);
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
bool decode_mfma_supported(const DecodeParams &p, int D, int kv_dtype, int batch);
int launch_decode_mfma(argus_hip_ctx *ctx, DecodeParams &p, int D, int batch, hipStream_t stream);
// Block-quantised caches (decode_blocks.hip): ARGUS_HIP_Q4_0 / Q4_1 / Q8_0, dequantised in registers.
int launch_decode_blocks(argus_hip_ctx *ctx, DecodeParams &p, int D, int kv_dtype, int batch, hipStream_t stream);

}  // namespace argus_decode
