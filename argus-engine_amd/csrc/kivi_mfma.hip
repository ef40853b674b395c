// KIVI fused dequant + decode attention on the matrix cores (Q2 / Q4 / Q8, head_dim 64 / 128 / 256).
//
// Same arithmetic as kivi_attn.hip (dequant `code*d + m`, crates/techniques/kivi/src/kivi_attn.cu:
// 213-218, block layouts kivi_attn.cu:256-262 / 357-361), reorganised so the per-code work is a
// mask, not `Hq/Hkv` FMAs:
//
//   logits  S[t][h] = sum_ch code[ch][t] * (q[h][ch] * d[ch])  +  sum_ch m[ch] * q[h][ch]
//   output  O[h][c] = sum_t (p[h][t] * d[t][cb]) * code[t][c]   +  sum_t p[h][t] * m[t][cb]
//
// The code sums are 16x16x32 f16 MFMAs.  The codes are the operand with 8 contraction values per
// lane (8 channels of one token for the logits, 8 tokens of one channel for the output); KIVI
// stores K per channel and V per token, i.e. both transposed relative to that, so each wave copies
// its unit's K and V tiles (32 tokens) into a private LDS region and gathers code bytes from there.
//
//  * A code field masked out of its byte *is* an f16 operand: an integer n < 1024 in the low bits
//    of a half is the subnormal n * 2^-24, which the MFMA multiplies exactly.  No conversion; the
//    field's bit position and the 2^-24 come back as one power-of-two factor on the result.
//  * One byte (two for Q8) holds the codes of two neighbouring tokens (K) or channels (V).  A lane
//    owns both: rows 2r and 2r+1 of the logits go to two accumulators fed from the same read.
//  * The block scales ride on the other operand: q*d as f16 hi + lo (the logits keep ~2^-22
//    relative accuracy, the 1e-4 bound on emitted scores needs it), and p*d in f16.  Only `group`
//    of the 16 operand columns are real heads, so the q*d work of a unit is spread over all 16
//    lanes of a row (each prepares one 32-channel slice for its head).  When the slice's MFMA is
//    issued the slice moves to the head's lanes with DPP row shifts, high halves into columns
//    0 .. GT-1 and low halves into columns GT .. 2GT-1 of one operand, so a single MFMA forms both
//    partial sums.  The p*d operands of the output sums do not move at all: each block's sums are
//    read from the accumulator rows of the lanes that prepared its operand.
//  * The zero-point terms: sum m*q on the vector ALU while the scales are read, sum p*m as one
//    more MFMA whose operand is the f16 `m` header itself.
//  * The softmax is computed once per logit: the 32 x GT sums of a unit move from the operand
//    columns to the lanes (bank, head) of their row first, a lane exponentiates 8 * GT / 16 values,
//    and the packed probabilities return to every lane of the head with DPP moves.  The maximum and
//    the zero-point dot product cross the wave's four rows with v_permlane16/32_swap.
//
// Waves are autonomous: a wave prefetches its next unit into registers while it works on the
// current one, and there is no workgroup barrier inside the unit loop.  The residual window (F32
// or F16 rows) is a second loop over the same MFMAs with the K rows split into f16 hi + lo.
#include "kivi_common.hpp"

#include <algorithm>
#include <type_traits>

namespace argus_kivi {

using namespace argus_decode;

namespace {

typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));

__device__ __forceinline__ void wave_lds_fence() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// Lane i of a 16-lane row takes the value of lane i + SHIFT (zero past the row end).
template <int SHIFT>
__device__ __forceinline__ uint32_t row_shl(uint32_t x) {
  if constexpr (SHIFT == 0) return x;
  else return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, 0x100 + SHIFT, 0xf, 0xf, true);
}
template <int SHIFT>
__device__ __forceinline__ half8_t row_shl(half8_t v) {
  u32x4_t w = __builtin_bit_cast(u32x4_t, v);
#pragma unroll
  for (int i = 0; i < 4; ++i) w[i] = row_shl<SHIFT>(w[i]);
  return __builtin_bit_cast(half8_t, w);
}
// Lanes of the banks (groups of 4 lanes) in BANKS take `src` from the lane the DPP control CTRL
// names (0x100 + n: lane i + n, 0x110 + n: lane i - n, 0xe4: the lane itself); the rest keep `old`.
template <int CTRL, int BANKS>
__device__ __forceinline__ half8_t dpp_merge(half8_t old, half8_t src) {
  u32x4_t o = __builtin_bit_cast(u32x4_t, old);
  const u32x4_t w = __builtin_bit_cast(u32x4_t, src);
#pragma unroll
  for (int i = 0; i < 4; ++i) o[i] = (uint32_t)__builtin_amdgcn_update_dpp((int)o[i], (int)w[i], CTRL, 0xf, BANKS, false);
  return __builtin_bit_cast(half8_t, o);
}
// Lanes of the banks in BANKS take `src` as it is; the rest keep `old`.
template <int BANKS>
__device__ __forceinline__ float bank_select(float old, float src) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, old), __builtin_bit_cast(int, src), 0xe4, 0xf, BANKS, false));
}
// Lanes of the banks in BANKS take `src` from the lane the DPP control names; the rest keep `old`.
template <int CTRL, int BANKS>
__device__ __forceinline__ uint32_t dpp_merge(uint32_t old, uint32_t src) {
  return (uint32_t)__builtin_amdgcn_update_dpp((int)old, (int)src, CTRL, 0xf, BANKS, false);
}
// The 16-lane row rotated by SHIFT lanes (used with SHIFT = 8 and with 4 then 8, where the sense
// of the rotation does not matter).
template <int SHIFT>
__device__ __forceinline__ float row_rot(float x) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x120 + SHIFT, 0xf, 0xf, true));
}
// op over the four 16-lane rows of the wave, result in every row: the row swaps of this target
// exchange odd and even rows (then the wave's halves) of two registers without going through LDS.
// (SWAP false: through LDS permutes, which measured 3-4 % faster for the 2-bit kernels at head_dim
// 64 and 128 and 1-4 % slower everywhere else.)
template <bool SWAP, typename OP>
__device__ __forceinline__ float reduce_rows(float x, OP op) {
  if constexpr (!SWAP) {
    x = op(x, __shfl_xor(x, 16, 64));
    return op(x, __shfl_xor(x, 32, 64));
  }
  const uint32_t b0 = __builtin_bit_cast(uint32_t, x);
  const auto s16 = __builtin_amdgcn_permlane16_swap(b0, b0, false, false);
  x = op(__builtin_bit_cast(float, (uint32_t)s16[0]), __builtin_bit_cast(float, (uint32_t)s16[1]));
  const uint32_t b1 = __builtin_bit_cast(uint32_t, x);
  const auto s32 = __builtin_amdgcn_permlane32_swap(b1, b1, false, false);
  return op(__builtin_bit_cast(float, (uint32_t)s32[0]), __builtin_bit_cast(float, (uint32_t)s32[1]));
}
template <int SHIFT>
__device__ __forceinline__ float row_shr_add(float x) {
  return x + __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x110 + SHIFT, 0xf, 0xf, true));
}
template <int SHIFT>
__device__ __forceinline__ float row_shl_add(float x) {
  if constexpr (SHIFT > 0 && SHIFT < 16) x += __builtin_bit_cast(float, row_shl<SHIFT>(__builtin_bit_cast(uint32_t, x)));
  return x;
}

// The lane's code field: 2*BITS bits holding two neighbouring codes (tokens 2r, 2r+1 of a K
// channel block, channels 2r, 2r+1 of a V token block).
template <int BITS>
__device__ __forceinline__ int field_offset(int r) {
  return 4 + (BITS == 8 ? 2 * r : BITS == 4 ? r : (r >> 1));
}
// Reads of two consecutive contraction slots, packed into the two halves of one word.  (Loads
// into the high half of a register do not keep the low half on this target, so the pair is
// packed with a byte permute.)
template <int BITS>
__device__ __forceinline__ uint32_t field_read2(const uint8_t *p0, const uint8_t *p1) {
  typedef uint16_t u16x2_t __attribute__((ext_vector_type(2)));
  u16x2_t t;
  if constexpr (BITS == 8) {
    t[0] = *(const uint16_t *)p0;
    t[1] = *(const uint16_t *)p1;
  } else {
    t[0] = *p0;
    t[1] = *p1;
  }
  return __builtin_bit_cast(uint32_t, t);
}
__device__ __forceinline__ uint32_t half_read2(const uint8_t *p0, const uint8_t *p1) {
  typedef uint16_t u16x2_t __attribute__((ext_vector_type(2)));
  u16x2_t t;
  t[0] = *(const uint16_t *)p0;
  t[1] = *(const uint16_t *)p1;
  return __builtin_bit_cast(uint32_t, t);
}
// Packed pair word -> the f16x2 operand words of the two codes of the field.
// The matrix core multiplies subnormal halves exactly but keeps product bits relative to the
// operand's exponent, not its leading one: a field in the lowest mantissa bits loses that many bits
// of the sum (measured: 2^-20 relative for a 4-bit field at bit 0, 2^-24 at bit 4).  The logits need
// the full f32 accuracy, so with PRECISE every field is first moved up to end at mantissa bit 7 or
// 9 (`presh`: that left shift, lane-dependent for Q2, whose field sits in either nibble of its
// byte); the output sums do not, and take the fields where they are.
template <int BITS, bool PRECISE>
__device__ __forceinline__ void field_pair(uint32_t v, int presh, uint32_t &w0, uint32_t &w1) {
  if constexpr (BITS == 8) {
    w0 = v & 0x00ff00ffu;
    w1 = __builtin_amdgcn_perm(v, v, 0x0c030c01u);  // [v.b1, 0, v.b3, 0]
  } else if constexpr (BITS == 4) {
    // Without PRECISE the second operand is the whole byte, 16 * high nibble + low nibble, still an
    // exact small integer: its sums minus the low nibbles' sums are 16 times the high nibbles' sums,
    // taken once at the end (byte_sums_to_high) instead of one more mask per pair here.
    w0 = PRECISE ? ((v << 4) & 0x00f000f0u) : (v & 0x000f000fu);
    w1 = PRECISE ? (v & 0x00f000f0u) : v;
  } else if constexpr (PRECISE) {
    v <<= presh;
    w0 = v & 0x00c000c0u;
    w1 = v & 0x03000300u;
  } else {
    // presh = 6 (low nibble) or 2 (high nibble): masks 0x3 / 0xc shifted to the field's nibble
    const uint32_t m0 = (0x00c000c0u >> presh), m1 = (0x03000300u >> presh);
    w0 = v & m0;
    w1 = v & m1;
  }
}
// Bit position of code `which` (0 / 1) inside the operand half.
template <int BITS>
__host__ __device__ constexpr int field_shift(int which) {
  return BITS == 8 ? 0 : BITS == 4 ? 4 : 6 + 2 * which;
}
// Same for the fields of the output sums, which stay in place (Q2: on top of the lane's 2^-presh).
template <int BITS>
__host__ __device__ constexpr int field_shift_v(int which) {
  return BITS == 8 ? 0 : BITS == 4 ? 4 * which : 6 + 2 * which;
}

// 8 consecutive residual elements (16-byte aligned) as floats
__device__ __forceinline__ void load_row8(const float *p, float (&o)[8]) {
  const float4_t a = *(const float4_t *)p, b = *(const float4_t *)(p + 4);
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    o[e] = a[e];
    o[4 + e] = b[e];
  }
}
__device__ __forceinline__ void load_row8(const _Float16 *p, float (&o)[8]) {
  const half8_t a = *(const half8_t *)p;
#pragma unroll
  for (int e = 0; e < 8; ++e) o[e] = (float)a[e];
}

// f(integral_constant<int, 0>) ... f(integral_constant<int, N - 1>): slice indices must be constants
// (they select DPP shifts).
template <typename F, int... I>
__device__ __forceinline__ void static_for_impl(F &f, std::integer_sequence<int, I...>) {
  (f(std::integral_constant<int, I>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void static_for(F &&f) {
  static_for_impl(f, std::make_integer_sequence<int, N>{});
}

constexpr float kLn2 = 0.6931471805599453f;
// Power of two on the f16 operands that carry block scales: keeps the low halves of the hi + lo
// splits and small p*d products out of the f16 subnormal range.
constexpr float kOpScale = 64.0f;
constexpr float kCodeUnit = 16777216.0f;  // a raw code field n is the half n * 2^-24

// Query heads per KV head the kernel takes (bounds the merge area).
constexpr int kMaxGroup = 8;

// FASTK (Q4 without scores): the logits take the whole code byte as the operand of the even tokens
// and subtract the odd tokens' sums afterwards, like the output sums do.  The difference of two f32
// sums, one of them 17 times the size of the result, keeps ~2^-20 of it: plenty for the outputs (2e-3)
// and not enough for emitted scores (1e-4 on probabilities), which keep the shifted nibbles.
template <int BITS, int D, int GT, bool SOFTCAP, bool FASTK>
__global__ __launch_bounds__(256, (D == 256) ? 2 : 3) void kivi_mfma_kernel(const KiviParams kp) {
  constexpr int BB = 4 + 32 * BITS / 8;  // block bytes
  constexpr int KK = D / 32;             // 32-channel slices == V blocks per token
  constexpr int TILE_BYTES = D * BB;     // one K tile == one V tile
  constexpr int TILE_VEC = TILE_BYTES / 16;
  constexpr int NCH = (TILE_VEC + 63) / 64;
  // In LDS the V tile gets 16 bytes of padding after every 8 tokens: a lane group j reads tokens
  // 8j..8j+7, and the unpadded stride of 8 tokens is a multiple of 128 bytes for head_dim 128, which
  // would put groups j and j+2 on the same banks.
  constexpr int VPAD = 16;
  constexpr int V8_VEC = 8 * KK * BB / 16;  // 16-byte vectors per 8 tokens
  // ... and the K tile 16 bytes after every two slices: slices lie 32 blocks = 32 (mod 64) dwords
  // apart, so the lanes that read the headers of slices kk and kk + 2 in one instruction would
  // otherwise hit the same banks with different addresses.
  constexpr int K2_VEC = 2 * 32 * BB / 16;  // 16-byte vectors per two slices
  constexpr int KPADS = 16 * ((KK + 1) / 2);
  constexpr int WAVE_BYTES = 2 * TILE_BYTES + KPADS + 4 * VPAD;
  constexpr int MERGE_BYTES = 4 * kMaxGroup * (D + 4) * 4 + 4 * kMaxGroup * KK * 4 + 2 * 4 * 16 * 4;
  constexpr int SMEM = (4 * WAVE_BYTES > MERGE_BYTES) ? 4 * WAVE_BYTES : MERGE_BYTES;
  constexpr int NREP = 16 / GT;               // lanes of a row that share one head
  constexpr int NS = (KK + NREP - 1) / NREP;  // slices each lane prepares
  constexpr int CI = 4 / NREP;                // token pairs of a unit whose softmax a lane computes
  // Where a lane prepares a single V block, its headers are read whole (scale and zero point in one
  // word) and the lane's column collects that block's zero-point sum; with more blocks per lane,
  // picking the zero points for the column costs more than reading them again.
  constexpr bool kHeaderWords = NS == 1;
  constexpr bool kRowSwap = BITS != 2;
  static_assert(GT == 4 || GT == 8, "the lane roles below are written for 4 or 8 heads per row");
  __shared__ __attribute__((aligned(16))) uint8_t smem[SMEM];

  const DecodeParams &p = kp.d;
  // A GQA group wider than 8 is covered by several workgroups per KV head, 8 heads each (they re-read
  // the blocks; the reference kernel runs one block per query head whatever the ratio).
  const int split = blockIdx.x, kvh = blockIdx.y / p.head_chunks, b = blockIdx.z;
  const int hchunk = blockIdx.y % p.head_chunks;
  const int hbase = kvh * p.group + kMaxGroup * hchunk;  // first query head of this workgroup
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // keeps unit indices and tile addresses scalar
  const int j = lane >> 4, r = lane & 15;
  const int ra = r / GT, rh = r % GT;  // slice owner index and head of this lane during preparation
  const int G = min(kMaxGroup, p.group - kMaxGroup * hchunk);  // heads of this workgroup
  const int gpf = kp.res_cap / kUnit;
  const int q_units = kp.q_tokens / kUnit;

  uint8_t *sK = smem + wave * WAVE_BYTES;
  uint8_t *sV = sK + TILE_BYTES + KPADS;
  const uint8_t *sVj = sV + j * (8 * KK * BB + VPAD);  // this lane group's 8 tokens
  const uint8_t *qk_b = kp.qk + (int64_t)b * kp.qk_bs;
  const uint8_t *qv_b = kp.qv + (int64_t)b * kp.qv_bs;
  const float qscale = p.scale * 1.4426950408889634f * kOpScale;  // log2 domain

  // q of head rh for the slices this lane prepares: slice s -> channels 32*(ra + s*NREP) + 8j + e,
  // scaled and split into f16 hi + lo once, as packed pairs (channels e, e + 1)
  half2_t qh2[NS][4], ql2[NS][4];
#pragma unroll
  for (int s = 0; s < NS; ++s) {
    const int kk = ra + s * NREP;
    const bool ok = kk < KK && rh < G;
    const float *qp = p.q + (int64_t)b * p.q_bs + (int64_t)(hbase + min(rh, G - 1)) * D + 32 * min(kk, KK - 1) + 8 * j;
    float qv[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) qv[e] = qp[e];  // the address is clamped
    loaded8(qv);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      _Float16 hi, lo;
      split_f16(ok ? qv[e] * qscale : 0.0f, hi, lo);
      qh2[s][e / 2][e % 2] = hi;
      ql2[s][e / 2][e % 2] = lo;
    }
  }

  const int foff = field_offset<BITS>(r);
  const int presh = 6 - 4 * (r & 1);  // Q2 only: the lane's field is the low or the high nibble of its byte

  // o_acc[2cb + sub]: lane (j, n = r) reg i -> accumulator row 4j + i, channel 32cb + 2r + sub.  The
  // rows GT*a .. GT*a + GT-1 belong to the heads 0 .. GT-1 as seen by the lanes that prepare for slot
  // a = row / GT: block cb's sums are the ones in the rows of slot cb % NREP (its p*d operand is used
  // where it was prepared; the other rows of that product are nobody's).
  float4_t o_acc[2 * KK];
  float4_t m_acc = {0.0f, 0.0f, 0.0f, 0.0f};  // zero-point term: lane (j, n = cb) reg i -> head (4j + i) % GT
#pragma unroll
  for (int a = 0; a < 2 * KK; ++a) o_acc[a] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
  float m_run = kNegInf, l_run = 0.0f;

  // Online-softmax step for one unit.  The 32 x GT logits of a unit are spread over all 64 lanes: lane
  // (j, ra, rh) holds, for head rh, the CI token pairs 8j + 2(ra*CI + ii) + w.  In: t[w][ii] = logit
  // (log2 units).  Out: the probabilities of tokens 8j .. 8j+7 for head rh, relative to the running
  // maximum, in every lane of the head (row 16j + r of a p operand is head r % GT).
  const float inv_cap = SOFTCAP ? 1.0f / p.softcap : 0.0f;
  auto softmax_step = [&](float(&t)[2][CI], int tok0, int n_valid) -> half8_t {
    float mt = kNegInf;
#pragma unroll
    for (int ii = 0; ii < CI; ++ii)
#pragma unroll
      for (int w = 0; w < 2; ++w) {
        if constexpr (SOFTCAP) {
          // cap * tanh(logit / cap) on the natural-unit logit, back to log2 units; NaN stays NaN
          const float sv = t[w][ii];
          const float capped = softcap_tanh(sv * kLn2, p.softcap, inv_cap) * 1.4426950408889634f;
          t[w][ii] = (sv != sv) ? sv : capped;
        }
        if (8 * j + 2 * (ra * CI + ii) + w >= n_valid) t[w][ii] = kNegInf;
        mt = fmaxf(mt, t[w][ii]);  // a NaN logit propagates (the reference kernels have no guard)
      }
    if (p.scores && rh < G) {
      float *srow = p.scores + (int64_t)b * p.score_bs + (int64_t)(hbase + rh) * p.score_stride + tok0 + 8 * j + 2 * ra * CI;
#pragma unroll
      for (int ii = 0; ii < CI; ++ii)
#pragma unroll
        for (int w = 0; w < 2; ++w)
          if (8 * j + 2 * (ra * CI + ii) + w < n_valid) srow[2 * ii + w] = t[w][ii] * kLn2;
    }
    // the head's maximum over its lanes: the other banks of the row, then the other rows
    if constexpr (NREP >= 4) mt = fmaxf(mt, row_rot<GT>(mt));
    mt = fmaxf(mt, row_rot<8>(mt));
    mt = reduce_rows<kRowSwap>(mt, [](float a, float b) { return fmaxf(a, b); });
    const float m_new = fmaxf(m_run, mt);
    const float m_ref = (m_new == kNegInf) ? 0.0f : m_new;
    const float alpha = __builtin_amdgcn_exp2f(m_run - m_ref);
    m_run = m_new;
    uint32_t own[CI];
    float lsum = 0.0f;  // f32 sum of this lane's tokens: the emitted probabilities are normalised by it
#pragma unroll
    for (int ii = 0; ii < CI; ++ii) {
      half2_t pw;
#pragma unroll
      for (int w = 0; w < 2; ++w) {
        const float e = __builtin_amdgcn_exp2f(t[w][ii] - m_ref);  // NaN stays NaN
        lsum += e;
        pw[w] = (_Float16)e;
      }
      own[ii] = __builtin_bit_cast(uint32_t, pw);  // token pair ra*CI + ii
    }
    l_run = l_run * alpha + lsum;
    if (__builtin_amdgcn_ballot_w64(alpha != 1.0f && rh < G) != 0) {  // (lanes past the group hold nobody's maximum)
      // accumulator row 4j + i belongs to head (4j + i) % GT
      float al[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) al[i] = __shfl(alpha, (4 * j + i) % GT, 64);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
#pragma unroll
        for (int a = 0; a < 2 * KK; ++a) o_acc[a][i] *= al[i];
        m_acc[i] *= al[i];
      }
    }
    // every lane of the head collects the four token pairs
    u32x4_t pa;
    if constexpr (GT == 8) {
#pragma unroll
      for (int ii = 0; ii < 2; ++ii) {
        pa[ii] = dpp_merge<0x110 + 8, 0xc>(own[ii], own[ii]);      // lanes 8..15 take pair ii from lanes 0..7
        pa[2 + ii] = dpp_merge<0x100 + 8, 0x3>(own[ii], own[ii]);  // lanes 0..7 take pair 2 + ii from lanes 8..15
      }
    } else {
      const uint32_t ev = dpp_merge<0x110 + 4, 0xa>(own[0], own[0]);  // pair 0 in banks 0, 1; pair 2 in banks 2, 3
      const uint32_t od = dpp_merge<0x100 + 4, 0x5>(own[0], own[0]);  // pair 1 in banks 0, 1; pair 3 in banks 2, 3
      pa[0] = dpp_merge<0x110 + 8, 0xc>(ev, ev);
      pa[2] = dpp_merge<0x100 + 8, 0x3>(ev, ev);
      pa[1] = dpp_merge<0x110 + 8, 0xc>(od, od);
      pa[3] = dpp_merge<0x100 + 8, 0x3>(od, od);
    }
    return __builtin_bit_cast(half8_t, pa);
  };

  const int u_begin = split * kp.units_per_split;
  const int u_end = min(kp.units_total, u_begin + kp.units_per_split);
  const int uq_end = min(u_end, q_units);
  int u = u_begin + wave;

  // ================================ quantised units ===============================================
  u32x4_t pk[NCH], pv[NCH];
  // The unit to fetch next, as (flush, 32-token group inside the flush); stepped without divisions.
  int f_flush = u / gpf, f_gif = u % gpf;
  auto fetch = [&]() {
    const int64_t kblk = ((int64_t)f_flush * p.n_heads_kv * gpf + (int64_t)kvh * gpf + f_gif) * D;
    const int64_t vblk = (((int64_t)f_flush * p.n_heads_kv + kvh) * kp.res_cap + f_gif * kUnit) * KK;
    const u32x4_t *ksrc = (const u32x4_t *)(qk_b + kblk * BB);
    const u32x4_t *vsrc = (const u32x4_t *)(qv_b + vblk * BB);
#pragma unroll
    for (int c = 0; c < NCH; ++c) {
      const int i = lane + 64 * c;
      if (i < TILE_VEC) {
        pk[c] = __builtin_nontemporal_load(ksrc + i);
        pv[c] = __builtin_nontemporal_load(vsrc + i);
      }
    }
    f_gif += 4;
    while (f_gif >= gpf) {
      f_gif -= gpf;
      ++f_flush;
    }
  };
  if (u < uq_end) fetch();

  for (; u < uq_end; u += 4) {
    wave_lds_fence();  // the previous unit's reads are done
#pragma unroll
    for (int c = 0; c < NCH; ++c) {
      const int i = lane + 64 * c;
      if (i < TILE_VEC) {
        ((u32x4_t *)sK)[i + i / K2_VEC] = pk[c];
        ((u32x4_t *)sV)[i + i / V8_VEC] = pv[c];
      }
    }
    wave_lds_fence();
    if (u + 4 < uq_end) fetch();

    // ---- this lane's share of q*d (hi + lo) and of sum m*q ----------------------------------------
    half8_t own_h[NS], own_l[NS];
    float c0 = 0.0f;
#pragma unroll
    for (int s = 0; s < NS; ++s) {
      const int kk = min(ra + s * NREP, KK - 1);  // qf is zero where the slice does not exist
      // Two blocks' headers (d | m << 16) at a time, as packed pairs.  With q = qh + ql and d all
      // f16, hi = rn(qh * d) leaves a remainder qh * d - hi that is itself an f16 number (one fma),
      // so hi + lo = q * d to the rounding of lo: the ~2^-22 the f32 product split gave, from three
      // packed instructions per pair instead of two conversions, a product and a split per value.
#pragma unroll
      for (int pr = 0; pr < 4; ++pr) {
        const uint32_t h0 = *(const uint32_t *)(sK + (32 * kk + 8 * j + 2 * pr) * BB + 16 * (kk / 2));
        const uint32_t h1 = *(const uint32_t *)(sK + (32 * kk + 8 * j + 2 * pr + 1) * BB + 16 * (kk / 2));
        const half2_t dd = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(h1, h0, 0x05040100u));  // [d0, d1]
        const half2_t mm = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(h1, h0, 0x07060302u));  // [m0, m1]
        half2_t hi = dd * qh2[s][pr];
        asm("" : "+v"(hi));  // one rounded value for both uses
        const half2_t rem = __builtin_elementwise_fma(dd, qh2[s][pr], -hi);
        const half2_t lo = __builtin_elementwise_fma(dd, ql2[s][pr], rem);
        own_h[s][2 * pr] = hi[0];
        own_h[s][2 * pr + 1] = hi[1];
        own_l[s][2 * pr] = lo[0];
        own_l[s][2 * pr + 1] = lo[1];
        c0 = __builtin_amdgcn_fdot2(mm, qh2[s][pr], c0, false);
        c0 = __builtin_amdgcn_fdot2(mm, ql2[s][pr], c0, false);
      }
    }
    c0 = reduce_rows<kRowSwap>(c0, [](float a, float b) { return a + b; });
    if constexpr (NREP >= 4) c0 += row_rot<GT>(c0);
    c0 += row_rot<8>(c0);
    c0 *= 1.0f / kOpScale;  // every lane now holds sum_ch m[ch] q[rh][ch]

    // ---- logits: rows m = r -> tokens 2r (s[0]) and 2r + 1 (s[1]) ----------------------------------
    float4_t s[2];
    s[0] = s[1] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
    auto qk_slice = [&](auto kk_c) {
      constexpr int kk = decltype(kk_c)::value;
      uint32_t w0[4], w1[4];
#pragma unroll
      for (int pr = 0; pr < 4; ++pr) {
        const uint8_t *cp = sK + (32 * kk + 8 * j + 2 * pr) * BB + 16 * (kk / 2) + foff;
        // (FASTK: w0 = low nibbles in place ... unused; the byte and the high nibbles are the operands)
        if constexpr (FASTK) {
          const uint32_t v = field_read2<BITS>(cp, cp + BB);
          w0[pr] = v;                // 16 * code(2r + 1) + code(2r)
          w1[pr] = v & 0x00f000f0u;  // 16 * code(2r + 1)
        } else {
          field_pair<BITS, true>(field_read2<BITS>(cp, cp + BB), presh, w0[pr], w1[pr]);
        }
      }
      const half8_t a0 = __builtin_bit_cast(half8_t, u32x4_t{w0[0], w0[1], w0[2], w0[3]});
      const half8_t a1 = __builtin_bit_cast(half8_t, u32x4_t{w1[0], w1[1], w1[2], w1[3]});
      // Operand columns 0 .. GT-1 take the high halves of the heads' q*d, columns GT .. 2GT-1 the low
      // halves (the rest of the 16 columns are nobody's), so one MFMA per token set forms both
      // partial sums; they are added once the slices are through.  The slice was prepared by the
      // lanes ra*GT .. ra*GT+GT-1 of each row.
      constexpr int ra_k = kk % NREP;
      constexpr int kLoBanks = (GT == 4) ? 0x2 : 0xc;
      constexpr int kLoCtrl = (ra_k == 0) ? 0x110 + GT : (ra_k == 1) ? 0xe4 : 0x100 + (ra_k - 1) * GT;
      constexpr int kHiBanks = (GT == 4) ? 0x1 : 0x3;
      half8_t bq;
      if constexpr (ra_k == 1) bq = dpp_merge<0x100 + GT, kHiBanks>(own_l[kk / NREP], own_h[kk / NREP]);  // the low halves are in place
      else bq = dpp_merge<kLoCtrl, kLoBanks>(row_shl<ra_k * GT>(own_h[kk / NREP]), own_l[kk / NREP]);
      s[0] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a0, bq, s[0], 0, 0, 0);
      s[1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a1, bq, s[1], 0, 0, 0);
    };
    static_for<KK>(qk_slice);
    // Column h plus column GT + h is head h's sum; token pair i of it goes to the lanes (ra, rh) =
    // (i / CI, h), so that the softmax below is computed once per logit instead of once per column.
    float t[2][CI];
#pragma unroll
    for (int w = 0; w < 2; ++w) {
      if constexpr (GT == 8) {
#pragma unroll
        for (int ii = 0; ii < 2; ++ii)
          t[w][ii] = bank_select<0xc>(row_shl_add<8>(s[w][ii]), row_shr_add<8>(s[w][2 + ii]));
      } else {
        float y[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) y[i] = row_shl_add<4>(s[w][i]);  // lanes 0..3: the heads' sums
        uint32_t x = __builtin_bit_cast(uint32_t, y[0]);
        x = dpp_merge<0x110 + 4, 0x2>(x, __builtin_bit_cast(uint32_t, y[1]));
        x = dpp_merge<0x110 + 8, 0x4>(x, __builtin_bit_cast(uint32_t, y[2]));
        x = dpp_merge<0x110 + 12, 0x8>(x, __builtin_bit_cast(uint32_t, y[3]));
        t[w][0] = __builtin_bit_cast(float, x);
      }
    }
#pragma unroll
    for (int ii = 0; ii < CI; ++ii) {
      if constexpr (FASTK) t[0][ii] -= t[1][ii];  // byte sums -> the even tokens' sums, in units of 2^-24
      // undo the field position and the operand units
#pragma unroll
      for (int w = 0; w < 2; ++w)
        t[w][ii] = fmaf(t[w][ii], kCodeUnit / (kOpScale * (float)(1 << ((FASTK && w == 0) ? 0 : field_shift<BITS>(w)))), c0);
    }

    const half8_t pa_all = softmax_step(t, u * kUnit, kUnit);

    // ---- output: contraction slot e -> token 8j + e -------------------------------------------------
    // Like q*d, the p*d operand only has `group` real rows: every lane of the row has its head's
    // probabilities and scales them for the V blocks it owns.
    const half8_t pa_s = pa_all * (_Float16)kOpScale;
    half8_t pd_own[NS];
    u32x4_t mw = {0u, 0u, 0u, 0u};  // zero points of the block whose sum this lane's column collects
#pragma unroll
    for (int s2 = 0; s2 < NS; ++s2) {
      const int cb = min(ra + s2 * NREP, KK - 1);
      u32x4_t dw;
#pragma unroll
      for (int pr = 0; pr < 4; ++pr) {
        const uint8_t *dp = sVj + (2 * pr * KK + cb) * BB;
        if constexpr (kHeaderWords) {
          // whole headers (d | m << 16) of two tokens, like the K blocks' above
          const uint32_t h0 = *(const uint32_t *)dp, h1 = *(const uint32_t *)(dp + KK * BB);
          dw[pr] = __builtin_amdgcn_perm(h1, h0, 0x05040100u);
          mw[pr] = __builtin_amdgcn_perm(h1, h0, 0x07060302u);
        } else {
          dw[pr] = half_read2(dp, dp + KK * BB);
        }
      }
      pd_own[s2] = pa_s * __builtin_bit_cast(half8_t, dw);  // p * d[token][cb]
    }
    auto pv_block = [&](auto cb_c) {
      constexpr int cb = decltype(cb_c)::value;
      const half8_t pd = pd_own[cb / NREP];  // real in the rows of slot cb % NREP, where it was prepared
      uint32_t w0[4], w1[4];
#pragma unroll
      for (int pr = 0; pr < 4; ++pr) {
        const uint8_t *cp = sVj + (2 * pr * KK + cb) * BB + foff;
        field_pair<BITS, false>(field_read2<BITS>(cp, cp + KK * BB), presh, w0[pr], w1[pr]);
      }
      const half8_t b0 = __builtin_bit_cast(half8_t, u32x4_t{w0[0], w0[1], w0[2], w0[3]});
      const half8_t b1 = __builtin_bit_cast(half8_t, u32x4_t{w1[0], w1[1], w1[2], w1[3]});
      o_acc[2 * cb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(pd, b0, o_acc[2 * cb], 0, 0, 0);
      o_acc[2 * cb + 1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(pd, b1, o_acc[2 * cb + 1], 0, 0, 0);
    };
    static_for<KK>(pv_block);
    // zero-point term: sum_t p[h][t] m[t][cb], in column n = cb, or with whole-header reads in the
    // columns of the lanes ra = cb, which had block cb's headers anyway
    if constexpr (!kHeaderWords) {
      if (r < KK) {
#pragma unroll
        for (int pr = 0; pr < 4; ++pr) {
          const uint8_t *mp = sVj + (2 * pr * KK + r) * BB + 2;
          mw[pr] = half_read2(mp, mp + KK * BB);
        }
      }
    }
    m_acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(pa_all, __builtin_bit_cast(half8_t, mw), m_acc, 0, 0, 0);
  }

  // Q4: the second accumulator of a block holds the byte sums (see field_pair)
  if constexpr (BITS == 4) {
#pragma unroll
    for (int cb = 0; cb < KK; ++cb) o_acc[2 * cb + 1] -= o_acc[2 * cb];
  }
  // The code sums carry the field position and the operand units.
  const float v_unit = (BITS == 2) ? (float)(1 << presh) : 1.0f;  // Q2 fields sit 2^-presh below bit 6
#pragma unroll
  for (int cb = 0; cb < KK; ++cb) {
    o_acc[2 * cb] *= v_unit * (kCodeUnit / (kOpScale * (float)(1 << field_shift_v<BITS>(0))));
    o_acc[2 * cb + 1] *= v_unit * (kCodeUnit / (kOpScale * (float)(1 << field_shift_v<BITS>(1))));
  }

  // ================================ residual window ===============================================
  // Rows [kv_heads, res_cap, D], F32 or F16; same lane roles (rows 2r / 2r+1, columns 2r / 2r+1).
  auto residual_unit = [&](auto tag, int ru) {
    using RES_T = decltype(tag);
    const int n_valid = min(kUnit, kp.res_tokens - ru * kUnit);
    const int64_t rbase = (int64_t)b * kp.res_bs + (int64_t)kvh * kp.res_cap * D + (int64_t)ru * kUnit * D;
    const RES_T *rk = (const RES_T *)kp.res_k + rbase;
    const RES_T *rv = (const RES_T *)kp.res_v + rbase;
    // operand column r carries head r % GT: every bank of the row gets the head's logits
    const float *qp = p.q + (int64_t)b * p.q_bs + (int64_t)(hbase + min(rh, G - 1)) * D + 8 * j;
    float4_t s[2];
    s[0] = s[1] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
      half8_t qh, ql;
      float qv[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) qv[e] = qp[32 * kk + e];
      loaded8(qv);
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        _Float16 hi, lo;
        split_f16((rh < G) ? qv[e] * qscale : 0.0f, hi, lo);
        qh[e] = hi;
        ql[e] = lo;
      }
#pragma unroll
      for (int w = 0; w < 2; ++w) {
        const RES_T *row = rk + (int64_t)min(2 * r + w, n_valid - 1) * D + 32 * kk + 8 * j;
        float rowv[8];
        load_row8(row, rowv);
        half8_t ah, al;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          _Float16 hi, lo;
          split_f16(rowv[e], hi, lo);
          ah[e] = hi;
          al[e] = lo;
        }
        s[w] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ah, qh, s[w], 0, 0, 0);
        s[w] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ah, ql, s[w], 0, 0, 0);
        s[w] = __builtin_amdgcn_mfma_f32_16x16x32_f16(al, qh, s[w], 0, 0, 0);
      }
    }
    // bank ra keeps its token pairs
    float t[2][CI];
#pragma unroll
    for (int w = 0; w < 2; ++w) {
      if constexpr (GT == 8) {
#pragma unroll
        for (int ii = 0; ii < 2; ++ii) t[w][ii] = bank_select<0xc>(s[w][ii], s[w][2 + ii]) * (1.0f / kOpScale);
      } else {
        t[w][0] = bank_select<0x8>(bank_select<0x4>(bank_select<0x2>(s[w][0], s[w][1]), s[w][2]), s[w][3]) * (1.0f / kOpScale);
      }
    }
    // every slot's rows hold their head's probabilities: whichever rows a block's sums are read from
    // (see o_acc), the residual tokens are in them
    const half8_t pa_all = softmax_step(t, kp.q_tokens + ru * kUnit, n_valid);
#pragma unroll
    for (int cs = 0; cs < 2 * KK; ++cs) {
      half8_t bv;
#pragma unroll
      for (int e = 0; e < 8; ++e)
        bv[e] = (_Float16)(float)rv[(int64_t)min(8 * j + e, n_valid - 1) * D + 32 * (cs / 2) + 2 * r + (cs & 1)];
      o_acc[cs] = __builtin_amdgcn_mfma_f32_16x16x32_f16(pa_all, bv, o_acc[cs], 0, 0, 0);
    }
  };
  for (; u < u_end; u += 4) {
    if (kp.res_f16) residual_unit((_Float16)0, u - q_units);
    else residual_unit(0.0f, u - q_units);
  }

  // ---- merge: lane groups (row sum), then the 4 waves through LDS --------------------------------
  l_run += __shfl_xor(l_run, 16, 64);
  l_run += __shfl_xor(l_run, 32, 64);
  if constexpr (NREP >= 4) l_run = row_shl_add<2 * GT>(l_run);
  l_run = row_shl_add<GT>(l_run);  // lanes r < GT: the head's sum over the banks
  __syncthreads();  // every wave is done with its tile region
  float(*lds_acc)[kMaxGroup][D + 4] = (float(*)[kMaxGroup][D + 4]) smem;
  float(*lds_mt)[kMaxGroup][KK] = (float(*)[kMaxGroup][KK])(smem + 4 * kMaxGroup * (D + 4) * 4);
  float(*lds_m)[16] = (float(*)[16])(smem + 4 * kMaxGroup * (D + 4) * 4 + 4 * kMaxGroup * KK * 4);
  float(*lds_l)[16] = lds_m + 4;
  if (j == 0) {
    lds_m[wave][r] = m_run;
    lds_l[wave][r] = l_run;
  }
#pragma unroll
  for (int cb = 0; cb < KK; ++cb) {
    if ((4 * j) / GT == cb % NREP) {  // this lane group's accumulator rows are block cb's (see o_acc)
#pragma unroll
      for (int i = 0; i < 4; ++i)
        *(float2 *)&lds_acc[wave][(4 * j) % GT + i][32 * cb + 2 * r] = make_float2(o_acc[2 * cb][i], o_acc[2 * cb + 1][i]);
    }
  }
  // zero-point sums: row 4j + i < GT is head 4j + i, the column depends on how the headers were read
  const int m_cb = kHeaderWords ? ra : r;
  if (4 * j < GT && m_cb < KK && (!kHeaderWords || rh == 0)) {
#pragma unroll
    for (int i = 0; i < 4; ++i) lds_mt[wave][4 * j + i][m_cb] = m_acc[i];
  }
  __syncthreads();

  for (int idx = threadIdx.x; idx < G * D; idx += 256) {
    const int g = idx / D, c = idx % D;
    const int h = hbase + g;
    const float mm = fmaxf(fmaxf(lds_m[0][g], lds_m[1][g]), fmaxf(lds_m[2][g], lds_m[3][g]));
    const float m_ref = (mm == kNegInf) ? 0.0f : mm;
    float o = 0.0f, ll = 0.0f;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      const float f = __builtin_amdgcn_exp2f(lds_m[w][g] - m_ref);
      // waves that processed no unit carry m = -inf and zero sums (f = 0)
      o += (lds_acc[w][g][c] + lds_mt[w][g][c / 32]) * f;
      ll += lds_l[w][g] * f;
    }
    const int64_t pidx = ((int64_t)b * p.n_heads_q + h) * p.nsplit + split;
    p.ws_o[pidx * D + c] = o;
    if (c == 0) {
      p.ws_ml[pidx * 2 + 0] = mm * kLn2;  // partials go to the combine pass in natural-log units
      p.ws_ml[pidx * 2 + 1] = ll;
    }
  }
}

template <int BITS, int D>
int launch(argus_hip_ctx *ctx, KiviParams &kp, int batch, hipStream_t stream) {
  DecodeParams &p = kp.d;
  p.head_chunks = (p.group + kMaxGroup - 1) / kMaxGroup;
  const int pairs = p.n_heads_kv * p.head_chunks * batch;
  // One round of co-resident workgroups: a second, partly filled round would run at a fraction of
  // the occupancy the unit loop needs to hide its LDS and HBM latency.
  const int wgs_per_cu = std::min(argus_wgs_per_cu(ctx, kivi_mfma_kernel<BITS, D, 4, false, false>, 256, 0),
                                  argus_wgs_per_cu(ctx, kivi_mfma_kernel<BITS, D, 8, false, false>, 256, 0));
  const int slots = ctx->compute_units * wgs_per_cu;
  const int max_splits = (kp.units_total + 3) / 4;  // at least one unit per wave
  int nsplit = std::max(1, std::min({slots / pairs, max_splits, kMaxSplits}));
  kp.units_per_split = (kp.units_total + nsplit - 1) / nsplit;
  nsplit = (kp.units_total + kp.units_per_split - 1) / kp.units_per_split;
  p.nsplit = nsplit;
  p.direct = 0;
  const int rc = reserve_partials(ctx, p, batch, D);
  if (rc != ARGUS_HIP_OK) return rc;
  ctx->plan = argus_hip_decode_plan{nsplit, kp.units_per_split * kUnit, wgs_per_cu, 0, 2, 3, 0};
  const dim3 grid(nsplit, p.n_heads_kv * p.head_chunks, batch);
  KernelTimer timer(ctx, stream);
  const bool cap = p.softcap > 0.0f;
  constexpr bool kFast = BITS == 4;
  const bool fast = kFast && !p.scores;  // (soft-capped calls take the exact form as well)
  if (p.group <= 4 && cap) hipLaunchKernelGGL((kivi_mfma_kernel<BITS, D, 4, true, false>), grid, dim3(256), 0, stream, kp);
  else if (p.group <= 4 && fast) hipLaunchKernelGGL((kivi_mfma_kernel<BITS, D, 4, false, kFast>), grid, dim3(256), 0, stream, kp);
  else if (p.group <= 4) hipLaunchKernelGGL((kivi_mfma_kernel<BITS, D, 4, false, false>), grid, dim3(256), 0, stream, kp);
  else if (cap) hipLaunchKernelGGL((kivi_mfma_kernel<BITS, D, 8, true, false>), grid, dim3(256), 0, stream, kp);
  else if (fast) hipLaunchKernelGGL((kivi_mfma_kernel<BITS, D, 8, false, kFast>), grid, dim3(256), 0, stream, kp);
  else hipLaunchKernelGGL((kivi_mfma_kernel<BITS, D, 8, false, false>), grid, dim3(256), 0, stream, kp);
  timer.mark();
  ARGUS_HIP_CHECK(ctx, hipGetLastError());
  hipLaunchKernelGGL((decode_combine_kernel<NoFallback, D>), combine_grid(p, batch), dim3(256), 0, stream, p);
  ARGUS_HIP_CHECK(ctx, hipGetLastError());
  return ARGUS_HIP_OK;
}

template <int BITS>
int launch_dim(argus_hip_ctx *ctx, KiviParams &kp, int batch, hipStream_t stream) {
  switch (kp.head_dim) {
    case 64: return launch<BITS, 64>(ctx, kp, batch, stream);
    case 128: return launch<BITS, 128>(ctx, kp, batch, stream);
    default: return launch<BITS, 256>(ctx, kp, batch, stream);
  }
}

}  // namespace

bool kivi_mfma_supported(const KiviParams &kp) {
  if (kp.head_dim != 64 && kp.head_dim != 128 && kp.head_dim != 256) return false;
  // tiles are copied as 16-byte vectors
  if ((((uintptr_t)kp.qk | (uintptr_t)kp.qv) & 15) || (kp.qk_bs & 15) || (kp.qv_bs & 15)) return false;
  // residual rows are read as 16-byte vectors
  if ((((uintptr_t)kp.res_k | (uintptr_t)kp.res_v) & 15) || (kp.res_bs & 7)) return false;
  return true;
}

int launch_kivi_mfma(argus_hip_ctx *ctx, KiviParams &kp, int bits, int batch, hipStream_t stream) {
  switch (bits) {
    case 2: return launch_dim<2>(ctx, kp, batch, stream);
    case 4: return launch_dim<4>(ctx, kp, batch, stream);
    default: return launch_dim<8>(ctx, kp, batch, stream);
  }
}

}  // namespace argus_kivi
