// Causal GQA flash-attention prefill on the gfx950 matrix cores.
//
// Stands in for Backend::flash_attention_prefill (engine/src/backend.rs:1011-1027; CPU semantics
// engine/src/layers/attention.rs:78-351, CUDA behaviour model
// engine/src/backend/cuda_pc/kernels.cu:559-816): key c is visible to query row r iff
// c <= r + q_start_pos (and c + window > r + q_start_pos), q_start_pos = cache_seq_len - seq_len;
// fully masked rows give zeros.
//
// Design:
//  * v_mfma_f32_32x32x16_f16 throughout, in the transposed formulation
//        S^T = K . Q^T     (A = K rows from LDS, B = Q rows held in registers)
//        O^T = V^T . P^T   (A = V^T from LDS, B = P^T taken straight from the S^T accumulators)
//    so a lane owns one query column: the softmax runs over in-lane registers plus one
//    cross-half shuffle, the O rescale is a per-lane scalar, and P never goes through LDS.
//  * One wave = 32 query rows of one Q head.  Four waves -- HPW heads of one GQA group times 4/HPW
//    consecutive 32-row blocks -- share each K/V tile, staged once in LDS (both row major; the V^T
//    operand comes out of a transposing LDS read), so GQA multiplies neither HBM nor LDS-fill
//    traffic.  A workgroup is one such quartet, or two of them (KV groups) on alternate key tiles
//    of the same query block when the grid alone would leave one wave per SIMD.
//  * Tiles are fetched into registers ahead of the step that stages them, through bounds-checked
//    buffer loads; the logits MFMAs of tile t+1 overlap the exponentials of tile t.
//  * blockIdx is laid out so that consecutive workgroups hit different KV heads (one XCD / L2 per
//    KV head when there are 8 of them); a workgroup takes query tiles n-1-j then j, so all carry
//    the same number of key tiles.
#include "argus_hip_internal.hpp"

#include <cstdlib>
#include <type_traits>

namespace {

typedef float float16_t __attribute__((ext_vector_type(16)));
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));

struct PrefillParams {
  const void *q;
  const void *k;
  const void *v;
  void *out;
  int32_t n_heads_q, n_heads_kv, group;
  int32_t seq_len, cache_len, q_start, capacity, batch, window;
  int32_t n_qtiles, group_chunks;  // grid decomposition
  int32_t unpaired;                // one query tile per workgroup, longest first (else the pair n-1-j, j)
  int32_t q_f16, out_f16;
  // F32 caches take two passes over the same kernel: V rounded to f16 first, then (v_residual) the
  // rounding's remainder v - f16(v), whose output is added to the first pass's (accumulate).
  int32_t v_residual, accumulate;
  float scale_log2e;
};

// Transposing LDS read (ds_read_b64_tr_b16), see its use below.
__device__ __forceinline__ half4_t lds_read_tr16(const _Float16 *p) {
  typedef short short4_t __attribute__((ext_vector_type(4)));
  typedef __attribute__((address_space(3))) short4_t lds_short4_t;
  return __builtin_bit_cast(half4_t, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4_t *)p));
}

// dword 3 of a raw (untyped, unstrided) buffer descriptor on this target
constexpr int kBufferFlags = 0x00020000;
typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));

// 8 consecutive K or V elements as f16, read through a bounds-checked buffer descriptor
// (byte offsets: per-lane `voff`, wave-uniform `soff`); out-of-range chunks read as zero.
// `residual` (F32 rows only): what the f16 rounding leaves, x - f16(x), itself as f16.
template <typename KV_T>
__device__ __forceinline__ half8_t load_kv_chunk(__amdgpu_buffer_rsrc_t rsrc, uint32_t voff, uint32_t soff, bool residual);
template <>
__device__ __forceinline__ half8_t load_kv_chunk<_Float16>(__amdgpu_buffer_rsrc_t rsrc, uint32_t voff, uint32_t soff, bool) {
  return __builtin_bit_cast(half8_t, __builtin_amdgcn_raw_buffer_load_b128(rsrc, voff, soff, 0));
}
template <>
__device__ __forceinline__ half8_t load_kv_chunk<float>(__amdgpu_buffer_rsrc_t rsrc, uint32_t voff, uint32_t soff, bool residual) {
  const float4_t a = __builtin_bit_cast(float4_t, __builtin_amdgcn_raw_buffer_load_b128(rsrc, voff, soff, 0));
  const float4_t b = __builtin_bit_cast(float4_t, __builtin_amdgcn_raw_buffer_load_b128(rsrc, voff + 16, soff, 0));
  half8_t h;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const float x = e < 4 ? a[e] : b[e - 4];
    const _Float16 hi = (_Float16)x;
    // an infinite or NaN element keeps its value in the first pass and adds nothing in the second
    const float rest = x - (float)hi;
    h[e] = residual ? ((rest == rest && __builtin_fabsf(rest) < 65504.0f) ? (_Float16)rest : (_Float16)0.0f) : hi;
  }
  return h;
}
// 8 consecutive f32 query elements times `c`, rounded to f16
__device__ __forceinline__ half8_t load_q_f32(const float *p, float c) {
  const float4_t a = *(const float4_t *)p, b = *(const float4_t *)(p + 4);
  half8_t h;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    h[e] = (_Float16)(a[e] * c);
    h[4 + e] = (_Float16)(b[e] * c);
  }
  return h;
}
// 8 consecutive f16 query elements times `c`
__device__ __forceinline__ half8_t load_q_f16(const _Float16 *p, float c) {
  const half8_t r = *(const half8_t *)p;
  half8_t h;
#pragma unroll
  for (int e = 0; e < 8; ++e) h[e] = (_Float16)((float)r[e] * c);
  return h;
}

// The same as hi + lo (lo = the f16 nearest to what hi leaves; zero where that is not finite)
__device__ __forceinline__ void load_q_f32_split(const float *p, float c, half8_t &hi, half8_t &lo) {
  const float4_t a = *(const float4_t *)p, b = *(const float4_t *)(p + 4);
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    float x = (e < 4 ? a[e] : b[e - 4]) * c;
    asm("" : "+v"(x));  // one f32 product for both halves (no fused re-rounding)
    const _Float16 h = (_Float16)x;
    const float rest = x - (float)h;
    hi[e] = h;
    lo[e] = (rest == rest && __builtin_fabsf(rest) < 65504.0f) ? (_Float16)rest : (_Float16)0.0f;
  }
}

// Sizes of one staged K/V tile pair, shared by the kernel and the launcher.  NH = Q heads per wave:
// a wave that holds two heads takes tiles of half the keys, so its accumulators take the same room.
template <int D, int NH, int SUB>
struct PrefillTile {
#ifndef PF_BN128
#define PF_BN128 32
#endif
#ifndef PF_BN64
#define PF_BN64 64
#endif
  static constexpr int BN = NH == 2 ? 32 : (D < 128 ? PF_BN64 : D == 128 ? PF_BN128 : 32);  // keys per register tile (one pipeline step)
  static constexpr int BT = BN * SUB;                     // keys per staged tile (one barrier)
  static constexpr int KP = D + 8;                        // K tile row pitch (halfs)
  // V tile row pitch (halfs): an odd multiple of 16 dwords, so that the 4 rows x 32 bytes a
  // 16-lane group touches in one transposing read, and the neighbouring group's 32 bytes next to
  // them, all fall on different banks.
  static constexpr int VP = D + 32;
  static constexpr int HALFS = BT * KP + BT * VP;  // halfs per staged (K, V) tile pair
};

// An F32 cache is the all-F32 shape of the reference's CPU path: there the f16 roundings of Q, of K
// and of the probabilities each move an output by up to ~1e-3 on rows that see a handful of keys
// (a seeded draw at d 256, 31 keys: 0.9e-3 + 1.1e-3 + 0.6e-3 = 2.06e-3, over the 2e-3 bar).  In those
// instantiations a workgroup whose rows see at most kFewKeys keys adds the logits of the query's low
// f16 half (re-read and split per tile: no registers are kept for it); with more keys the errors
// average out and the workgroup runs as ever.  F16 caches (the reference's GPU shape and every
// benchmark configuration) are not touched.
template <typename KV_T>
constexpr bool kQueryLo = std::is_same<KV_T, float>::value;

// D head_dim; HPW head slots and WPG waves per KV group (WPG / HPW consecutive 32-row query blocks);
// NG KV groups; NH Q heads of the GQA group held by one wave (every K / V operand read from LDS then
// feeds NH MFMAs); SUB register tiles (pipeline steps) per staged tile, i.e. per barrier.
template <int D, int HPW, int WPG, int NG, typename KV_T, int NH, int SUB>
#ifndef PF_OCC64
#define PF_OCC64 2
#endif
__global__ __launch_bounds__(64 * WPG * NG, (WPG * NG == 4 && D <= 128) ? ((D == 64 && NH == 1) ? PF_OCC64 : 2) : 1) void prefill_kernel(const PrefillParams p) {
  using TL = PrefillTile<D, NH, SUB>;
  static_assert(SUB == 1 || SUB == 2, "one or two register tiles per staged tile");
  constexpr bool QLO = kQueryLo<KV_T>;
  static_assert(!QLO || NH == 1, "the low query half is only carried by one-head waves");
  constexpr int kFewKeys = 128;
  constexpr int BN = TL::BN, BT = TL::BT, KP = TL::KP, VP = TL::VP;
  constexpr int NT = 64 * WPG * NG;          // threads
  constexpr int QPW = WPG / HPW;             // 32-row query blocks per workgroup
  constexpr int KK = D / 16;                 // MFMA k-steps over head_dim
  constexpr int KB = BN / 32;                // S^T row blocks (32 keys each)
  constexpr int RB = D / 32;                 // O^T row blocks (32 channels each)
  constexpr int CH = NG * BT * D / 8 / NT;   // 16-byte chunks per thread per iteration
  static_assert(CH >= 1 && CH * NT * 8 == NG * BT * D, "tile chunks must divide over the threads");
  constexpr int kLdsAhead = 4;               // MFMA operand reads kept in flight
#ifndef PF_VAHEAD64
#define PF_VAHEAD64 4
#endif
  constexpr int kVAhead = (D <= 64) ? PF_VAHEAD64 : 3;
#ifndef PF_VALU_MASK
#define PF_VALU_MASK 0x402
#endif
#ifndef PF_PHASE_VALU
#define PF_PHASE_VALU ((D <= 64) ? 4 : (D == 128 && BN == 32) ? 3 : 0)
#endif
  constexpr int kPhaseValu = PF_PHASE_VALU;  // vector-ALU instructions placed behind each MFMA of a phase

  // [2 buffers][NG tiles][K tile | V^T tile]; reused at the end for the cross-group merge.
  extern __shared__ __attribute__((aligned(16))) _Float16 smem[];

  // ---- work decomposition ------------------------------------------------------------------
  const int pairs = p.batch * p.n_heads_kv;
  const int pair = blockIdx.x % pairs;
  const int j = blockIdx.x / pairs;
  const int b = pair / p.n_heads_kv, kvh = pair % p.n_heads_kv;
  const int gc = j % p.group_chunks;
  const int jt = j / p.group_chunks;

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int kvg = wave / WPG, wq = wave % WPG;  // KV group of this wave, query-wave index
  const int ln = lane & 31, hl = lane >> 5;
  const int h0 = kvh * p.group + (gc * HPW + (wq % HPW)) * NH;  // first of this wave's NH heads

  // Causal work grows linearly with the query tile index, so each workgroup takes the pair
  // (n_qtiles-1-jt, jt): every workgroup then carries the same number of key tiles.
  for (int pass = 0; pass < 2; ++pass) {
  const int qt = (pass == 0 || p.unpaired) ? (p.n_qtiles - 1 - jt) : jt;
  if (pass == 1 && (p.unpaired || qt == p.n_qtiles - 1 - jt)) break;
  const int qb = qt * QPW + wq / HPW;
  const int r0 = qb * 32;            // first query row of this wave
  const int row = r0 + ln;           // this lane's query row
  const bool row_ok = row < p.seq_len;

  // ---- Q as the B operand: lane (query ln, half hl) holds Q[row][16kk + 8hl .. +7] ----------
  half8_t qreg[NH][KK];
  // (QLO) the rows of this pass see few keys: the logits also take the query's low half
  const int keys_seen = min((qt + 1) * QPW * 32 + p.q_start, p.cache_len);  // by the last row of the pass
  const bool few_keys = QLO && !p.q_f16 && (p.window > 0 ? min(keys_seen, p.window) : keys_seen) <= kFewKeys;
  // Rows past seq_len re-read the last row (their columns are never stored), so the loads carry
  // no lane condition and are issued back to back.
  const int64_t qoff0 = (((int64_t)b * p.seq_len + min(row, p.seq_len - 1)) * p.n_heads_q + h0) * D + 8 * hl;
  auto load_q = [&]() {
#pragma unroll
    for (int n = 0; n < NH; ++n)
#pragma unroll
      for (int kk = 0; kk < KK; ++kk)
        qreg[n][kk] = p.q_f16 ? load_q_f16((const _Float16 *)p.q + qoff0 + n * D + 16 * kk, p.scale_log2e)
                              : load_q_f32((const float *)p.q + qoff0 + n * D + 16 * kk, p.scale_log2e);
  };

  float16_t o_acc[NH][RB];
#pragma unroll
  for (int n = 0; n < NH; ++n)
#pragma unroll
    for (int r = 0; r < RB; ++r)
#pragma unroll
      for (int i = 0; i < 16; ++i) o_acc[n][r][i] = 0.0f;
  // The query is held times scale * log2(e), and the logit accumulators start from -m_ref (negm: sixteen
  // copies of it, the shape of an accumulator block; m_ref = m_run, or 0 while the row has seen no key),
  // so the matrix cores deliver exponents ready for v_exp_f32.
  // (kFold; where registers allow.  Otherwise the accumulators start from zero and m_ref is
  // subtracted in front of the exponential.)
#ifndef PF_FOLD
#define PF_FOLD (D <= 64 || (D == 128 && BN == 32))
#endif
  constexpr bool kFold = PF_FOLD;
  float m_run[NH], l_run[NH], m_ref[NH];
  float16_t negm[NH];
#pragma unroll
  for (int n = 0; n < NH; ++n) {
    m_run[n] = kNegInf, l_run[n] = 0.0f, m_ref[n] = 0.0f;
    if constexpr (kFold) {
#pragma unroll
      for (int i = 0; i < 16; ++i) negm[n][i] = 0.0f;
    }
  }

  // ---- key range of the workgroup -----------------------------------------------------------
  const int wg_row_last = min(p.seq_len, (qt + 1) * QPW * 32) - 1;
  const int kv_end = min(p.cache_len, wg_row_last + p.q_start + 1);
  int kv_begin = 0;
  if (p.window > 0) kv_begin = max(0, qt * QPW * 32 + p.q_start - p.window + 1);
  const int kt_begin = kv_begin / BT, kt_end = (kv_end + BT - 1) / BT;
  const int n_it = (kt_end - kt_begin + NG - 1) / NG;

  const KV_T *kbase = (const KV_T *)p.k + ((int64_t)b * p.n_heads_kv + kvh) * p.capacity * D;
  const KV_T *vbase = (const KV_T *)p.v + ((int64_t)b * p.n_heads_kv + kvh) * p.capacity * D;

  // Iteration `it` covers tiles kt_begin + it*NG + g for g < NG (tile g is consumed by KV group g).
  // Software pipeline inside each wave: the S^T MFMAs of iteration it+1 are issued before the
  // softmax of iteration it, so the matrix core works while the vector ALU does the exponentials.
  // That needs K one iteration further ahead than V: K tiles are staged two iterations ahead into
  // sKb[it & 1], V^T tiles one ahead into sVb[it & 1]; in iteration `it` the waves read
  // sKb[(it+1) & 1] and sVb[it & 1] and fill sKb[it & 1] and sVb[(it+1) & 1], so one barrier per
  // iteration still separates every fill from the reads before and after it.
  _Float16 *const sKb = smem;                         // [2][NG][BT * KP]
  _Float16 *const sVb = smem + 2 * NG * BT * KP;      // [2][NG][BT * VP]
  // kDeep: tiles are fetched one step earlier than they are staged (two register sets, alternating
  // by step parity), so a fetch has a whole extra step to arrive; used where registers allow.
#ifndef PF_DEEP128
#define PF_DEEP128 1
#endif
  constexpr bool kDeep = (D <= 64 && NH == 1 && SUB == 1) || (PF_DEEP128 && D == 128 && SUB == 1 && !QLO);
  half8_t kpre[kDeep ? 2 : 1][CH], vpre[kDeep ? 2 : 1][CH];
  // Chunk cid of an iteration's NG tiles is the 16 bytes at element 8*cid from the first tile's
  // first row (the tiles are adjacent in the cache), so a fetch is a scalar tile offset plus a
  // per-thread constant.  The loads go through a buffer descriptor that ends at the last visible
  // key: rows past it come back as zeros from the bounds check, with no branch and no address
  // arithmetic, and every step issues the same number of loads, which lets the compiler wait for
  // exactly the loads a staging step needs and leave the younger ones in flight.
  const uint32_t kv_bytes = (uint32_t)kv_end * D * sizeof(KV_T);
  const __amdgpu_buffer_rsrc_t k_rsrc = __builtin_amdgcn_make_buffer_rsrc((void *)kbase, 0, kv_bytes, kBufferFlags);
  const __amdgpu_buffer_rsrc_t v_rsrc = __builtin_amdgcn_make_buffer_rsrc((void *)vbase, 0, kv_bytes, kBufferFlags);
  auto fetch_tiles = [&](__amdgpu_buffer_rsrc_t rsrc, int it, half8_t(&pre)[CH], bool residual) {
    const uint32_t tile_off = (uint32_t)((kt_begin + it * NG) * BT) * (D * sizeof(KV_T));
#pragma unroll
    for (int c = 0; c < CH; ++c)
      pre[c] = load_kv_chunk<KV_T>(rsrc, (uint32_t)(threadIdx.x + NT * c) * (8 * sizeof(KV_T)), tile_off, residual);
  };
  auto fetch_k = [&](int it, auto set_c) { fetch_tiles(k_rsrc, it, kpre[decltype(set_c)::value], false); };
  auto fetch_v = [&](int it, auto set_c) { fetch_tiles(v_rsrc, it, vpre[decltype(set_c)::value], p.v_residual != 0); };
  auto stage_k = [&](int buf, auto set_c) {
    constexpr int SET = decltype(set_c)::value;
#pragma unroll
    for (int c = 0; c < CH; ++c) {
      const int cid = threadIdx.x + NT * c;
      const int trow = cid / (D / 8), dc = cid % (D / 8);
      const int g = trow / BT, key = trow % BT;
      *(half8_t *)(sKb + (buf * NG + g) * (BT * KP) + key * KP + 8 * dc) = kpre[SET][c];
    }
  };
  auto stage_v = [&](int buf, auto set_c) {
    constexpr int SET = decltype(set_c)::value;
#pragma unroll
    for (int c = 0; c < CH; ++c) {
      const int cid = threadIdx.x + NT * c;
      const int trow = cid / (D / 8), dc = cid % (D / 8);
      const int g = trow / BT, key = trow % BT;
      *(half8_t *)(sVb + (buf * NG + g) * (BT * VP) + key * VP + 8 * dc) = vpre[SET][c];
    }
  };

  // Does this wave have anything to do with its tile of iteration `it`?
  const int wave_hi = r0 + 31 + p.q_start;  // largest visible key of the wave
  const int wave_lo = p.window > 0 ? (r0 + p.q_start - p.window + 1) : 0;
  // (register tile u of the staged tile of iteration it)
  auto tile_active = [&](int it, int u) {
    const int kt = kt_begin + it * NG + kvg;
    const int key0 = kt * BT + u * BN;
    return it < n_it && kt < kt_end && r0 < p.seq_len && key0 <= wave_hi && key0 + BN > wave_lo && key0 < kv_end;
  };
  // Instruction order of a phase, given once all of its code has been emitted (the groups only draw on
  // instructions in front of them): operand reads kept a few MFMAs ahead (one LDS round trip is
  // several times an MFMA's 32 cycles), and behind every MFMA NV of the phase's vector-ALU
  // instructions -- the exponentials of another tile -- because a wave issues in order and MFMAs back
  // to back would hold them up until the last has started.
  auto sched_qk = [&](auto nv_c) {
    constexpr int NV = decltype(nv_c)::value;
    constexpr int AH = kLdsAhead < KK * KB ? kLdsAhead : KK * KB;
    __builtin_amdgcn_sched_group_barrier(0x100, AH, 0);
#pragma unroll
    for (int i = 0; i < KK * KB; ++i) {
#pragma unroll
      for (int n = 0; n < NH; ++n) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        if (n == 0 && i < KK * KB - AH) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        if constexpr (NV > 0) __builtin_amdgcn_sched_group_barrier(PF_VALU_MASK, NV, 0);
      }
    }
  };
  auto sched_pv = [&](auto nv_c) {  // two transposing reads per operand
    constexpr int NV = decltype(nv_c)::value;
    constexpr int AH = kVAhead < (BN / 16) * RB ? kVAhead : (BN / 16) * RB;
    __builtin_amdgcn_sched_group_barrier(0x100, 2 * AH, 0);
#pragma unroll
    for (int i = 0; i < (BN / 16) * RB; ++i) {
#pragma unroll
      for (int n = 0; n < NH; ++n) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        if (n == 0 && i < (BN / 16) * RB - AH) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
        if constexpr (NV > 0) __builtin_amdgcn_sched_group_barrier(PF_VALU_MASK, NV, 0);
      }
    }
  };
  // S^T = K . Q^T for this wave's tile of iteration `it`
  typedef float16_t STile[NH][KB];
  auto qk_tile = [&](int it, int u, STile &s_acc, bool hints = true) {
    const _Float16 *sK = sKb + ((it & 1) * NG + kvg) * (BT * KP) + u * (BN * KP);
#pragma unroll
    for (int kk = 0; kk < KK; ++kk)
#pragma unroll
      for (int kb = 0; kb < KB; ++kb) {
        const half8_t a = *(const half8_t *)(sK + (32 * kb + ln) * KP + 16 * kk + 8 * hl);
#pragma unroll
        for (int n = 0; n < NH; ++n) {
          if (kFold && kk == 0)
            s_acc[n][kb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, qreg[n][kk], negm[n], 0, 0, 0);
          else if (kk == 0)
            s_acc[n][kb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, qreg[n][kk], float16_t{0.0f}, 0, 0, 0);
          else
            s_acc[n][kb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, qreg[n][kk], s_acc[n][kb], 0, 0, 0);
        }
      }
    if (hints) sched_qk(std::integral_constant<int, 0>{});
    if constexpr (QLO) {
      if (few_keys) {  // uniform over the workgroup
#pragma unroll
        for (int kk = 0; kk < KK; ++kk) {
          half8_t hi, lo;
          load_q_f32_split((const float *)p.q + qoff0 + 16 * kk, p.scale_log2e, hi, lo);
#pragma unroll
          for (int kb = 0; kb < KB; ++kb) {
            const half8_t a = *(const half8_t *)(sK + (32 * kb + ln) * KP + 16 * kk + 8 * hl);
            s_acc[0][kb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, lo, s_acc[0][kb], 0, 0, 0);
          }
          __builtin_amdgcn_sched_barrier(0);  // one slice's query registers at a time: this path is rare and must not cost the common one registers
        }
      }
    }
  };
  // Mask (edge tiles only) and row maximum of the tile of iteration `it`, whose accumulators hold
  // logit - m_ref.  The reference only moves when a row's maximum exceeds it by more than kLazy (log2
  // units), or when the row sees its first key: the tile's exponents, the accumulator start values
  // and m_run move at once, and the factor the running sums must take before this tile is added is
  // returned (1 for almost every tile).
  constexpr float kLazy = 8.0f;
  auto row_max = [&](float16_t(&s_acc)[KB]) {
    float mt = kNegInf;
#pragma unroll
    for (int kb = 0; kb < KB; ++kb)
#pragma unroll
      for (int i = 0; i < 16; ++i) mt = fmaxf(mt, s_acc[kb][i]);
    return xor32_combine(mt, [](float a, float b) { return fmaxf(a, b); });
  };
  // exponents of a tile whose accumulators were formed against the old reference follow it
  auto shift_tile = [&](float16_t(&s_acc)[KB], float delta) {
    if constexpr (kFold) {
#pragma unroll
      for (int kb = 0; kb < KB; ++kb)
#pragma unroll
        for (int i = 0; i < 16; ++i) s_acc[kb][i] -= delta;
    }
  };
  auto shift_ref = [&](int n, float delta) {  // m_ref += delta (a no-op in lanes whose delta is zero)
    if constexpr (kFold) {
#pragma unroll
      for (int i = 0; i < 16; ++i) negm[n][i] -= delta;
    }
    m_ref[n] += delta;
  };
  typedef float Alpha[NH];
  auto mask_max = [&](int it, int u, STile &s_acc, Alpha &alpha) {
    const int key0 = (kt_begin + it * NG + kvg) * BT + u * BN;
    const int q_pos = row + p.q_start;
    const bool need_mask = (key0 + BN - 1 > r0 + p.q_start) || (key0 + BN > p.cache_len) ||
                           (p.window > 0 && key0 < r0 + 31 + p.q_start - p.window + 1);
    if (need_mask) {
      const int lo = p.window > 0 ? q_pos - p.window : -1;  // keys <= lo are outside the window
      const int hi = min(q_pos, p.cache_len - 1);
#pragma unroll
      for (int kb = 0; kb < KB; ++kb)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int key = key0 + 32 * kb + 8 * (i / 4) + 4 * hl + (i % 4);
          const bool vis = key <= hi && key > lo;
#pragma unroll
          for (int n = 0; n < NH; ++n) s_acc[n][kb][i] = vis ? s_acc[n][kb][i] : kNegInf;
        }
    }
#pragma unroll
    for (int n = 0; n < NH; ++n) {
      const float mt = row_max(s_acc[n]) - (kFold ? 0.0f : m_ref[n]);
      const bool first = m_run[n] == kNegInf;
      const float delta = first ? (mt == kNegInf ? 0.0f : mt) : (mt > kLazy ? mt : 0.0f);
      alpha[n] = first ? 0.0f : __builtin_amdgcn_exp2f(-delta);
      if (__builtin_amdgcn_ballot_w64(delta != 0.0f) != 0) {
        shift_tile(s_acc[n], delta);
        shift_ref(n, delta);
      }
      if (!first || mt != kNegInf) m_run[n] = m_ref[n];
    }
  };
  auto rescale = [&](int n, float alpha) {
    if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0) {
#pragma unroll
      for (int r = 0; r < RB; ++r)
#pragma unroll
        for (int i = 0; i < 16; ++i) o_acc[n][r][i] *= alpha;
      l_run[n] *= alpha;
    }
  };
  typedef half8_t PTile[NH][BN / 16];
  // probabilities of P^T slices [J0, J1) of a tile (16 keys each) into pt; returns their row sum
  auto exp_part = [&](int n, float16_t(&s_acc)[KB], half8_t(&pt)[BN / 16], auto j0_c, auto j1_c) -> float {
    // The row sum is taken over the f16-rounded probabilities the matrix cores consume, so the
    // rounding cancels in the final normalisation.
    float lsum = 0.0f;
#pragma unroll
    for (int jn = decltype(j0_c)::value; jn < decltype(j1_c)::value; ++jn) {
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float x = s_acc[jn / 2][8 * (jn % 2) + e];
        pt[jn][e] = (_Float16)__builtin_amdgcn_exp2f(kFold ? x : x - m_ref[n]);
      }
#pragma unroll
      for (int e = 0; e < 8; e += 2) {
        const half2_t pr = {pt[jn][e], pt[jn][e + 1]}, one = {(_Float16)1.0f, (_Float16)1.0f};
        lsum = __builtin_amdgcn_fdot2(pr, one, lsum, false);
      }
    }
    return lsum;
  };
  typedef std::integral_constant<int, 0> J0;
  typedef std::integral_constant<int, BN / 16> JN;
  // Interior steps form the first kSplit slices of a tile's probabilities one phase early (beside
  // the output MFMAs of the tile before), so both phases of a step carry vector-ALU work.
#ifndef PF_SPLIT
#define PF_SPLIT ((D <= 64) ? BN / 32 : (D == 128 && BN == 32) ? 1 : 0)
#endif
  constexpr int kSplit = PF_SPLIT;
  typedef std::integral_constant<int, kSplit> JS;
  // Interior tiles take no maximum: the exponents stand against a reference that some earlier tile
  // of the row set, and a probability only leaves f16's range when a logit exceeds that reference
  // by 16 -- which shows in the tile's row sum.  Then (rarely) the reference moves up to the tile's
  // maximum: the sums so far, this tile's exponents and the next tile's (already formed against the
  // old reference) are corrected and the probabilities taken again.
  auto overflow_fix = [&](int n, float16_t(&s_cur)[KB], float16_t(&s_next)[KB], half8_t(&pt)[BN / 16]) -> float {
    const float mt = row_max(s_cur) - (kFold ? 0.0f : m_ref[n]);
    const float delta = mt > kLazy ? mt : 0.0f;
    rescale(n, __builtin_amdgcn_exp2f(-delta));
    shift_tile(s_cur, delta);
    shift_tile(s_next, delta);
    shift_ref(n, delta);
    m_run[n] = m_ref[n];
    return exp_part(n, s_cur, pt, J0{}, JN{});
  };
  // O^T += V^T . P^T for the tile of iteration `it`.
  // V stays row major in LDS.  The A operand wants, per lane, 8 keys of one channel:
  // ds_read_b64_tr_b16 delivers exactly that transposition.  In a group of 16 lanes, lane 4q + c
  // receives element c of the 8-byte rows addressed by lanes q, 4 + q, 8 + q, 12 + q; with lane s
  // addressing V[key0 + s / 4][ch0 + 4 (s % 4) ..], lane i gets channel ch0 + i of keys key0 ..
  // key0 + 3.  Lane groups 0..3 are (channels 0-15 | 16-31) x (lane half 0 | 1); P^T has keys
  // 4 hl + {0..3} and 8 + 4 hl + {0..3} of each 16 in the contraction slots of lane half hl.
  const int g16 = lane >> 4, s16 = lane & 15;
  const int vlane_off = (4 * (g16 >> 1) + (s16 >> 2)) * VP + 16 * (g16 & 1) + 4 * (s16 & 3);
  auto pv_tile = [&](int it, int u, PTile &pb, bool hints = true) {
    const _Float16 *vlane = sVb + ((it & 1) * NG + kvg) * (BT * VP) + u * (BN * VP) + vlane_off;
#pragma unroll
    for (int jn = 0; jn < BN / 16; ++jn)
#pragma unroll
      for (int r = 0; r < RB; ++r) {
        const _Float16 *vp = vlane + (16 * jn) * VP + 32 * r;
        const half4_t lo = lds_read_tr16(vp), hi = lds_read_tr16(vp + 8 * VP);
        const half8_t a = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
#pragma unroll
        for (int n = 0; n < NH; ++n) o_acc[n][r] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, pb[n][jn], o_acc[n][r], 0, 0, 0);
      }
    if (hints) sched_pv(std::integral_constant<int, 0>{});
  };

  // One pipeline step.  On entry s_cur holds the exponents of iteration `it`.  Phase A issues the
  // logits MFMAs of iteration it+1 while the vector ALU exponentiates tile `it`; phase B issues the
  // output MFMAs of tile `it` while the vector ALU starts on tile it+1 (its first exponentials in an
  // interior step, its mask and maximum otherwise).  Interior steps (every tile of the iteration
  // lies below the diagonal of every wave, inside the cache and the window, and there is a next
  // iteration) have no per-wave conditions, so each phase is one basic block the scheduler can
  // interleave.
  // Probabilities, rounded to f16 in P^T operand order: of the current tile, and (interior steps)
  // the first slices of the next one.
  PTile pb_a, pb_b;
  float l_head[NH];  // row sums of the slices formed early
#pragma unroll
  for (int n = 0; n < NH; ++n) l_head[n] = 0.0f;
  // (u_c: which register tile of the staged tile; the tile's fetches are issued with its first register
  // tile, its staging and the barrier follow its last)
  auto step = [&](int it, auto u_c, STile &s_cur, STile &s_next, PTile &pb_cur, PTile &pb_next, Alpha &a_cur,
                  auto interior_c, auto parity_c) {
    constexpr bool INTERIOR = decltype(interior_c)::value;
    constexpr int U = decltype(u_c)::value;
    constexpr bool LAST = U == SUB - 1;
    // register set fetched into during this step, and the one staged at its end
    typedef std::integral_constant<int, kDeep ? decltype(parity_c)::value : 0> FetchSet;
    typedef std::integral_constant<int, kDeep ? 1 - decltype(parity_c)::value : 0> StageSet;
    constexpr int AHEAD = kDeep ? 1 : 0;
    const int it_n = LAST ? it + 1 : it;  // the register tile after this one
    constexpr int U_N = LAST ? 0 : U + 1;
    const bool act = INTERIOR || tile_active(it, U);
    const bool has_next = INTERIOR || it_n < n_it;
    if (!INTERIOR && act) {  // its branches stay out of the phases below
#pragma unroll
      for (int n = 0; n < NH; ++n) rescale(n, a_cur[n]);
    }
    if constexpr (U == 0) {
      fetch_k(it + 2 + AHEAD, FetchSet{});  // past the last tile: all zeros, nothing is read
      fetch_v(it + 1 + AHEAD, FetchSet{});
    }
    // ---- phase A
    if (has_next) qk_tile(it_n, U_N, s_next, !INTERIOR);  // harmless on a tile the wave cannot see
    if constexpr (INTERIOR) {
      float lsum[NH];
      bool over = false;
#pragma unroll
      for (int n = 0; n < NH; ++n) {
        lsum[n] = l_head[n] + exp_part(n, s_cur[n], pb_cur[n], JS{}, JN{});
        over = over || !(lsum[n] < 1e30f);
      }
      sched_qk(std::integral_constant<int, kPhaseValu>{});
      if (__builtin_amdgcn_ballot_w64(over) != 0) {
#pragma unroll
        for (int n = 0; n < NH; ++n)
          if (__builtin_amdgcn_ballot_w64(!(lsum[n] < 1e30f)) != 0) lsum[n] = overflow_fix(n, s_cur[n], s_next[n], pb_cur[n]);
      }
#pragma unroll
      for (int n = 0; n < NH; ++n) l_run[n] += lsum[n];
    } else {
      if (act) {
#pragma unroll
        for (int n = 0; n < NH; ++n) l_run[n] += exp_part(n, s_cur[n], pb_cur[n], J0{}, JN{});
      }
    }
    // ---- phase B
    if (act) pv_tile(it, U, pb_cur, !INTERIOR);
    if constexpr (INTERIOR) {
#pragma unroll
      for (int n = 0; n < NH; ++n) {
        l_head[n] = exp_part(n, s_next[n], pb_next[n], J0{}, JS{});
        a_cur[n] = 1.0f;
      }
      sched_pv(std::integral_constant<int, kPhaseValu>{});
    } else {
      if (tile_active(it_n, U_N)) mask_max(it_n, U_N, s_next, a_cur);
    }
    if constexpr (LAST) {
      if (INTERIOR || it + 2 < n_it) stage_k(it & 1, StageSet{});  // a fill nobody reads is harmless
      if (has_next) stage_v((it + 1) & 1, StageSet{});
      __syncthreads();  // fills are visible; every wave is done with the buffers the next step refills
    }
  };

  STile s_a, s_b;
  {
    typedef std::integral_constant<int, 0> Set0;
    typedef std::integral_constant<int, kDeep ? 1 : 0> Set1;
    // Tiles past the last one read as zeros, so nothing here depends on n_it.  The query rows are
    // requested behind the first tiles and arrive with them.
    fetch_k(0, Set0{});
    fetch_v(0, Set0{});
    if constexpr (kDeep) fetch_k(1, Set1{});  // second register set: all three first tiles in one round trip
    __builtin_amdgcn_sched_barrier(0);
    load_q();
    stage_k(0, Set0{});
    stage_v(0, Set0{});
    if constexpr (!kDeep) fetch_k(1, Set0{});
    stage_k(1, Set1{});
    if constexpr (kDeep) {  // what step 0 stages at its end
      fetch_k(2, Set1{});
      fetch_v(1, Set1{});
    }
  }
  __syncthreads();
  Alpha t_cur;
#pragma unroll
  for (int n = 0; n < NH; ++n) t_cur[n] = 1.0f;
  if (n_it > 0) qk_tile(0, 0, s_a);
  if (tile_active(0, 0)) mask_max(0, 0, s_a, t_cur);
  if constexpr (SUB == 1) __syncthreads();  // sKb[0] is refilled by the first step
  // leading interior iterations (with one register tile per staged tile: rounded down to pairs, so
  // that s_a holds the current logits after them)
  int n_int = 0;
  if (p.window == 0) {
    const int full_keys = min(qt * QPW * 32 + p.q_start + 1, p.cache_len);  // keys every row of the workgroup sees
    n_int = max(0, min(n_it - 1, (full_keys / BT - kt_begin) / NG - 1));
    if (SUB == 1) n_int &= ~1;
  }
  // All loads issued so far have landed before the steady state begins: the waits inside the loop
  // then only ever concern the loads of the loop itself and can leave the youngest in flight.
  __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0)
  typedef std::integral_constant<int, 0> U0;
  typedef std::integral_constant<int, 1> U1;
  int it = 0;
  if (n_int > 0) {
#pragma unroll
    for (int n = 0; n < NH; ++n) l_head[n] = exp_part(n, s_a[n], pb_a[n], J0{}, JS{});
  }
  if constexpr (SUB == 1) {
    for (; it < n_int; it += 2) {
      step(it, U0{}, s_a, s_b, pb_a, pb_b, t_cur, std::true_type{}, U0{});
      step(it + 1, U0{}, s_b, s_a, pb_b, pb_a, t_cur, std::true_type{}, U1{});
    }
  } else {
    for (; it < n_int; ++it) {
      step(it, U0{}, s_a, s_b, pb_a, pb_b, t_cur, std::true_type{}, U0{});
      step(it, U1{}, s_b, s_a, pb_b, pb_a, t_cur, std::true_type{}, U0{});
    }
  }
  // the tile the interior steps leave behind has its exponents but no maximum yet (and the slices of
  // its probabilities formed early are formed again with the others)
  if (it > 0) mask_max(it, 0, s_a, t_cur);
  if constexpr (SUB == 1) {
    for (; it < n_it; it += 2) {
      step(it, U0{}, s_a, s_b, pb_a, pb_a, t_cur, std::false_type{}, U0{});
      if (it + 1 < n_it) step(it + 1, U0{}, s_b, s_a, pb_a, pb_a, t_cur, std::false_type{}, U1{});
    }
  } else {
    for (; it < n_it; ++it) {
      step(it, U0{}, s_a, s_b, pb_a, pb_a, t_cur, std::false_type{}, U0{});
      step(it, U1{}, s_b, s_a, pb_a, pb_a, t_cur, std::false_type{}, U0{});
    }
  }

  // ---- merge the KV groups through LDS, normalise and store --------------------------------------
  // Two groups trade halves: each hands the other (m, l) and one half of its O^T row blocks, merges
  // the half it keeps and stores it, so both do half the LDS traffic, half the arithmetic and half
  // the stores of a one-sided merge and neither waits for the other to finish.
  constexpr bool kTradeHalves = NG == 2 && RB % 2 == 0;
  if constexpr (kTradeHalves) {
#pragma unroll
    for (int n = 0; n < NH; ++n) l_run[n] += __shfl_xor(l_run[n], 32, 64);
    constexpr int KEEP = RB / 2;  // row blocks a group ends up with
    float *mrg = (float *)smem;   // [2 senders][WPG query waves][NH][KEEP*16 + 2][64 lanes]
    constexpr int SLOTS = KEEP * 16 + 2;
    auto hand_over = [&](auto first_c) {  // row blocks [FIRST, FIRST + KEEP) go to the other group
      constexpr int FIRST = decltype(first_c)::value;
#pragma unroll
      for (int n = 0; n < NH; ++n) {
        float *dst = mrg + ((kvg * WPG + wq) * NH + n) * SLOTS * 64 + lane;
#pragma unroll
        for (int r = 0; r < KEEP; ++r)
#pragma unroll
          for (int i = 0; i < 16; ++i) dst[(r * 16 + i) * 64] = o_acc[n][FIRST + r][i];
        dst[KEEP * 16 * 64] = m_run[n];
        dst[(KEEP * 16 + 1) * 64] = l_run[n];
      }
    };
    // ... the other group's [FIRST, FIRST + KEEP) are merged into this one's, normalised and stored
    // (lane = query row, registers = channels)
    auto take_and_store = [&](auto first_c) {
      constexpr int FIRST = decltype(first_c)::value;
#pragma unroll
      for (int n = 0; n < NH; ++n) {
        const float *src = mrg + (((1 - kvg) * WPG + wq) * NH + n) * SLOTS * 64 + lane;
        const float m_o = src[KEEP * 16 * 64], l_o = src[(KEEP * 16 + 1) * 64];
        const float m_new = fmaxf(m_run[n], m_o);
        const float m_to = (m_new == kNegInf) ? 0.0f : m_new;
        const float fa = __builtin_amdgcn_exp2f(m_run[n] - m_to), fb = __builtin_amdgcn_exp2f(m_o - m_to);
        const float l_all = l_run[n] * fa + l_o * fb;
        const float inv = l_all > 0.0f ? 1.0f / l_all : 0.0f;
        const int64_t ooff = (((int64_t)b * p.seq_len + row) * p.n_heads_q + h0 + n) * D;
#pragma unroll
        for (int r = 0; r < KEEP; ++r)
#pragma unroll
          for (int i4 = 0; i4 < 4; ++i4) {
            float4_t o;
#pragma unroll
            for (int e = 0; e < 4; ++e) o[e] = (o_acc[n][FIRST + r][4 * i4 + e] * fa + src[(r * 16 + 4 * i4 + e) * 64] * fb) * inv;
            const int d0 = 32 * (FIRST + r) + 8 * i4 + 4 * hl;
            if (!row_ok) continue;
            if (p.out_f16) {
              half4_t oh = {(_Float16)o[0], (_Float16)o[1], (_Float16)o[2], (_Float16)o[3]};
              *(half4_t *)((_Float16 *)p.out + ooff + d0) = oh;
            } else {
              float4_t *dst = (float4_t *)((float *)p.out + ooff + d0);
              if (p.accumulate) o += *dst;
              *dst = o;
            }
          }
      }
    };
    typedef std::integral_constant<int, 0> Lower;
    typedef std::integral_constant<int, KEEP> Upper;
    if (kvg == 0) hand_over(Upper{});
    else hand_over(Lower{});
    __syncthreads();
    if (kvg == 0) take_and_store(Lower{});
    else take_and_store(Upper{});
  } else {
  // ---- merge the KV groups: groups > 0 hand (m, l, O^T) to group 0 through LDS ---------------
#pragma unroll
  for (int n = 0; n < NH; ++n) l_run[n] += __shfl_xor(l_run[n], 32, 64);
  if constexpr (NG > 1) {
    float *mrg = (float *)smem;  // [NG-1][WPG query waves][NH][RB*16 + 2][64 lanes]
    constexpr int SLOTS = RB * 16 + 2;
    if (kvg > 0) {
#pragma unroll
      for (int n = 0; n < NH; ++n) {
        float *dst = mrg + (((kvg - 1) * WPG + wq) * NH + n) * SLOTS * 64 + lane;
#pragma unroll
        for (int r = 0; r < RB; ++r)
#pragma unroll
          for (int i = 0; i < 16; ++i) dst[(r * 16 + i) * 64] = o_acc[n][r][i];
        dst[RB * 16 * 64] = m_run[n];
        dst[(RB * 16 + 1) * 64] = l_run[n];
      }
    }
    __syncthreads();
    if (kvg == 0) {
#pragma unroll
    for (int g = 1; g < NG; ++g)
#pragma unroll
      for (int n = 0; n < NH; ++n) {
        const float *src = mrg + (((g - 1) * WPG + wq) * NH + n) * SLOTS * 64 + lane;
        const float m_o = src[RB * 16 * 64], l_o = src[(RB * 16 + 1) * 64];
        const float m_new = fmaxf(m_run[n], m_o);
        const float m_to = (m_new == kNegInf) ? 0.0f : m_new;
        const float fa = __builtin_amdgcn_exp2f(m_run[n] - m_to), fb = __builtin_amdgcn_exp2f(m_o - m_to);
#pragma unroll
        for (int r = 0; r < RB; ++r)
#pragma unroll
          for (int i = 0; i < 16; ++i) o_acc[n][r][i] = o_acc[n][r][i] * fa + src[(r * 16 + i) * 64] * fb;
        l_run[n] = l_run[n] * fa + l_o * fb;
        m_run[n] = m_new;
      }
    }
  }

  // ---- normalise and store: lane = query row, registers = channels ---------------------------
  if (row_ok && kvg == 0) {
#pragma unroll
  for (int n = 0; n < NH; ++n) {
  const float inv = l_run[n] > 0.0f ? 1.0f / l_run[n] : 0.0f;
  const int64_t ooff = (((int64_t)b * p.seq_len + row) * p.n_heads_q + h0 + n) * D;
#pragma unroll
  for (int r = 0; r < RB; ++r)
#pragma unroll
    for (int i4 = 0; i4 < 4; ++i4) {
      const int d0 = 32 * r + 8 * i4 + 4 * hl;
      float4_t o = {o_acc[n][r][4 * i4] * inv, o_acc[n][r][4 * i4 + 1] * inv, o_acc[n][r][4 * i4 + 2] * inv,
                    o_acc[n][r][4 * i4 + 3] * inv};
      if (p.out_f16) {
        half4_t oh = {(_Float16)o[0], (_Float16)o[1], (_Float16)o[2], (_Float16)o[3]};
        *(half4_t *)((_Float16 *)p.out + ooff + d0) = oh;
      } else {
        float4_t *dst = (float4_t *)((float *)p.out + ooff + d0);
        if (p.accumulate) o += *dst;
        *dst = o;
      }
    }
  }
  }
  }
  __syncthreads();  // the merge area is free again before the next pass stages tiles into it
  }  // pass
}

template <int D, int HPW, int WPG, int NG, typename KV_T, int NH, int SUB>
int launch_ng(argus_hip_ctx *ctx, PrefillParams &p, hipStream_t stream) {
  using TL = PrefillTile<D, NH, SUB>;
  constexpr int QPW = WPG / HPW;
  p.n_qtiles = (p.seq_len + 32 * QPW - 1) / (32 * QPW);
  p.group_chunks = p.group / (HPW * NH);
  // Workgroups take the query tiles in pairs (n-1-j, j) of equal total length, which balances a grid
  // that is resident all at once.  A grid of four or more workgroups per CU is balanced by the order
  // of dispatch instead: one tile per workgroup, longest first, and a workgroup's start-up runs beside
  // its neighbours' loops (d 64, 16K tokens: 1,045 against 1,065-1,085 us; at 512 workgroups and
  // below the pairs are 2-3 % faster).
  const int64_t paired = (int64_t)p.batch * p.n_heads_kv * p.group_chunks * ((p.n_qtiles + 1) / 2);
  p.unpaired = paired >= 4 * (int64_t)ctx->compute_units;
  const int64_t wgs = p.unpaired ? (int64_t)p.batch * p.n_heads_kv * p.group_chunks * p.n_qtiles : paired;
  if (wgs > 0x7fffffff) return argus_fail(ctx, ARGUS_HIP_ERR_UNSUPPORTED, "prefill: grid too large");
  // two buffers of NG tile pairs; the merge of the KV groups reuses the space
  size_t lds_bytes = 2 * NG * (size_t)TL::HALFS * sizeof(_Float16);
  // (two groups trade halves of their row blocks, each with its (m, l); more hand whole rows to group 0)
  const size_t merge_bytes = (NG == 2 ? (size_t)2 * WPG * NH * (D / 64 * 16 + 2) : (size_t)(NG - 1) * WPG * NH * (D / 32 * 16 + 2)) * 64 * sizeof(float);
  if (merge_bytes > lds_bytes) lds_bytes = merge_bytes;
  if (lds_bytes > ctx->props.sharedMemPerBlock)
    return argus_fail(ctx, ARGUS_HIP_ERR_UNSUPPORTED, "prefill: %zu bytes of LDS needed, %zu available", lds_bytes,
                      (size_t)ctx->props.sharedMemPerBlock);
  auto kern = prefill_kernel<D, HPW, WPG, NG, KV_T, NH, SUB>;
  if (lds_bytes > 48 * 1024) ARGUS_HIP_CHECK(ctx, argus_raise_lds_limit(ctx, kern, (int)lds_bytes));
  {
    KernelTimer timer(ctx, stream);
    hipLaunchKernelGGL(kern, dim3((unsigned)wgs), dim3(64 * WPG * NG), lds_bytes, stream, p);
  }
  ARGUS_HIP_CHECK(ctx, hipGetLastError());
  return 1;  // dispatched
}

// Workgroups a launch of this decomposition would have.
template <int HPW, int WPG, int NH>
int64_t prefill_wgs(const PrefillParams &p) {
  constexpr int QPW = WPG / HPW;
  const int64_t n_qtiles = (p.seq_len + 32 * QPW - 1) / (32 * QPW);
  return (int64_t)p.batch * p.n_heads_kv * (p.group / (HPW * NH)) * ((n_qtiles + 1) / 2);
}

template <int D, int HPW, typename KV_T>
int launch(argus_hip_ctx *ctx, PrefillParams &p, hipStream_t stream) {
  // Two waves per SIMD are needed to overlap anything.  When the grid alone provides them -- two
  // 4-wave workgroups per compute unit -- the workgroups run independently and measure 4-8 % faster
  // (S >= 4096 at Hq32/Hkv8).  Smaller grids get them from two KV groups inside an 8-wave workgroup:
  // the groups take alternate key tiles of the same query block and merge at the end (the 2K-token, head_dim 64
  // prefill shape: 32.3 us against 33.9 us).  Four groups would need a 128-VGPR cap that spills.
  const int64_t fill = 2 * (int64_t)ctx->compute_units;
#ifndef PF_SUB128
#define PF_SUB128 1
#endif
  constexpr int kSub = (D == 128 && std::is_same<KV_T, _Float16>::value) ? PF_SUB128 : 1;
  if constexpr (D <= 128) {
    // (F32 cache at head_dim 128: the four-wave form spills half as much again as the eight-wave one)
    const bool grid_fills = prefill_wgs<HPW, 4, 1>(p) >= fill && !(kQueryLo<KV_T> && D == 128);
    if (!grid_fills) return launch_ng<D, HPW, 4, 2, KV_T, 1, kSub>(ctx, p, stream);
  }
  return launch_ng<D, HPW, 4, 1, KV_T, 1, kSub>(ctx, p, stream);
}

// Two Q heads per wave (F16 caches at head_dim 64, even GQA groups, no window): every K / V operand
// read from LDS feeds two MFMAs.  Used where such workgroups (two head pairs x two query blocks) still
// fill the device twice over: 16K tokens at Hq32/Hkv8 take 1,107 against 1,215 us.  Smaller grids would
// need their second wave per SIMD from more KV groups of two waves each, and that form measured slower
// than one head per wave (2K tokens: 38.5 against 29.3 us).  Two register tiles per staged tile -- half
// the barriers -- were also built (the SUB parameter): 1,213 against 1,226 us without the folded
// accumulator start values, and with them the allocator spills, so tiles are staged one at a time.
#ifndef PF_PAIR
#define PF_PAIR 1
#endif
template <int HPW>
bool pair_fills(argus_hip_ctx *ctx, const PrefillParams &p) {
  return PF_PAIR && p.window == 0 && prefill_wgs<HPW, 4, 2>(p) >= 2 * (int64_t)ctx->compute_units;
}

template <int D, typename KV_T>
int dispatch_heads(argus_hip_ctx *ctx, PrefillParams &p, hipStream_t stream) {
  if constexpr (D == 64 && std::is_same<KV_T, _Float16>::value) {
    if (p.group % 4 == 0 && pair_fills<2>(ctx, p)) return launch_ng<64, 2, 4, 1, _Float16, 2, 1>(ctx, p, stream);
    if (p.group % 4 != 0 && p.group % 2 == 0 && pair_fills<1>(ctx, p)) return launch_ng<64, 1, 4, 1, _Float16, 2, 1>(ctx, p, stream);
  }
  if (p.group % 4 == 0) return launch<D, 4, KV_T>(ctx, p, stream);
  if (p.group % 2 == 0) return launch<D, 2, KV_T>(ctx, p, stream);
  return launch<D, 1, KV_T>(ctx, p, stream);
}

template <typename KV_T>
int dispatch_dim(argus_hip_ctx *ctx, PrefillParams &p, int D, hipStream_t stream) {
  switch (D) {
    case 64: return dispatch_heads<64, KV_T>(ctx, p, stream);
    case 128: return dispatch_heads<128, KV_T>(ctx, p, stream);
    default: return dispatch_heads<256, KV_T>(ctx, p, stream);
  }
}

}  // namespace

ARGUS_API int argus_hip_flash_attention_prefill(argus_hip_ctx *ctx, const argus_hip_prefill_args *a) {
  if (!ctx || !a) return ARGUS_HIP_ERR_INVALID;
  if (!a->q || !a->k_cache || !a->v_cache || !a->out)
    return argus_fail(ctx, ARGUS_HIP_ERR_INVALID, "flash_attention_prefill: null tensor pointer");
  if (a->n_heads_q <= 0 || a->n_heads_kv <= 0 || a->n_heads_q % a->n_heads_kv)
    return argus_fail(ctx, ARGUS_HIP_ERR_INVALID, "flash_attention_prefill: heads %d/%d", a->n_heads_q, a->n_heads_kv);
  if (a->seq_len <= 0 || a->batch_size <= 0 || a->cache_seq_len < a->seq_len || a->cache_seq_len > a->kv_capacity ||
      a->window < 0)
    return argus_fail(ctx, ARGUS_HIP_ERR_INVALID, "flash_attention_prefill: seq_len %d cache_seq_len %d capacity %d",
                      a->seq_len, a->cache_seq_len, a->kv_capacity);
  // Declined cases: the caller runs its CPU path (same set as cuda_pc.rs:851-860).
  if (!a->is_head_major) return 0;
  if (a->head_dim != 64 && a->head_dim != 128 && a->head_dim != 256) return 0;
  if (a->kv_dtype != ARGUS_HIP_F16 && a->kv_dtype != ARGUS_HIP_F32) return 0;
  if ((a->q_dtype != ARGUS_HIP_F16 && a->q_dtype != ARGUS_HIP_F32) ||
      (a->out_dtype != ARGUS_HIP_F16 && a->out_dtype != ARGUS_HIP_F32))
    return 0;
  if (((uintptr_t)a->q | (uintptr_t)a->k_cache | (uintptr_t)a->v_cache | (uintptr_t)a->out) & 15)
    return argus_fail(ctx, ARGUS_HIP_ERR_INVALID, "flash_attention_prefill: tensors must be 16-byte aligned");

  // K/V tiles are addressed with 32-bit byte offsets from the head's first row
  const size_t kv_elem = a->kv_dtype == ARGUS_HIP_F16 ? 2 : 4;
  if (((size_t)a->kv_capacity + 1024) * a->head_dim * kv_elem > 0xffffffffull)
    return argus_fail(ctx, ARGUS_HIP_ERR_UNSUPPORTED, "flash_attention_prefill: one head's cache (%d rows) exceeds 4 GiB",
                      a->kv_capacity);

  PrefillParams p{};
  p.q = a->q;
  p.k = a->k_cache;
  p.v = a->v_cache;
  p.out = a->out;
  p.n_heads_q = a->n_heads_q;
  p.n_heads_kv = a->n_heads_kv;
  p.group = a->n_heads_q / a->n_heads_kv;
  p.seq_len = a->seq_len;
  p.cache_len = a->cache_seq_len;
  p.q_start = a->cache_seq_len - a->seq_len;
  p.capacity = a->kv_capacity;
  p.batch = a->batch_size;
  p.window = a->window;
  p.q_f16 = a->q_dtype == ARGUS_HIP_F16;
  p.out_f16 = a->out_dtype == ARGUS_HIP_F16;
  p.scale_log2e = 1.4426950408889634f / sqrtf((float)a->head_dim);
  hipStream_t stream = (hipStream_t)a->stream;
  if (a->kv_dtype == ARGUS_HIP_F16) return dispatch_dim<_Float16>(ctx, p, a->head_dim, stream);
  // F32 cache: the matrix cores take f16 operands.  Rounding K moves a logit by ~1e-4 (nothing at the
  // 2e-3 output bar), but rounding V moves an output that one key dominates by up to 2^-12 |v|, 2e-3
  // for |v| >= 4: over the bar in a few rows per thousand random cases.  A second pass over the same
  // logits with V's rounding remainder restores the f32 values (F32 outputs; an F16 output rounds by
  // more than that itself).
  // (one timing bracket over both launches: an F32 cache with F32 output costs two passes)
  KernelTimer both(ctx, stream);
  struct Hold {
    argus_hip_ctx *c;
    ~Hold() { c->timer_held = false; }
  } hold{ctx};
  ctx->timer_held = true;
  const int rc = dispatch_dim<float>(ctx, p, a->head_dim, stream);
  if (rc != 1 || p.out_f16) return rc;
  p.v_residual = 1;
  p.accumulate = 1;
  return dispatch_dim<float>(ctx, p, a->head_dim, stream);
}
