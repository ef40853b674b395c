// Split-KV flash-decode over block-quantised caches (q4_0, q4_1, q8_0), dequantised in registers.
//
// The Q4_0 arm of Backend::attention_gen (engine/src/backend/cpu/common.rs:676-850: dequantise each
// K / V row, then the F32 algorithm with its NaN and uniform-weights guards) and the in-kernel form
// of the `--kv-format` attention whose reference floor decodes the whole cache to F32 first
// (engine/src/kv/standard_format.rs:538-643).  Blocks are the descriptor formats of
// engine/src/format/dtype_layout.rs:102-166 with 32 elements: [f16 d][f16 m?][codes];
// q4_0: x = d * (n - 8), q4_1: x = d * n + m, n = 4-bit code, element i in the low nibble of code
// byte i, element 16 + i in the high nibble; q8_0: x = d * c, c = int8.
//
// Same data flow as decode_mfma.hip (nothing goes through LDS memory).  A lane turns the 4 (q4) or
// 8 (q8) code bytes it loaded into 8 f16 values: v_perm puts each code under the exponent of 1024
// and a packed subtract leaves the exact integer.
//   S^T[token][head] = sum over blocks kk of d_kk(token) * (C_kk . Q_kk^T)
//       v_mfma_f32_16x16x32_f16 per 32-element block with A = the integer codes n - 8 (q4_0), n
//       (q4_1) or c (q8_0) -- lane (j, r) = token r, code bytes 4j..4j+3 of block kk, i.e. elements
//       {4j..4j+3, 16+4j..16+4j+3} (q8: elements 8j..8j+7) -- and B = the same elements of Q as
//       f16 hi + lo, so the block dot products are exact to f32.  The scale is applied to the MFMA
//       result: the result lane (j, h) holds tokens 4j..4j+3, whose scales sit in lanes 20j + i of
//       the wave and are fetched with ds_bpermute (q4_1 adds m_kk(token) * sum of Q_kk).  Logits
//       therefore carry no f16 rounding of d * (n - 8), and the emitted scores keep the 1e-4 bar.
//   O[head][channel] = P . V     v_mfma_f32_16x16x16_f16
//       B: lane (j, r) loads, for tokens 4j..4j+3, code bytes 4(r%4).. of block r/4, dequantises
//       them to f16 (one rounding, 2^-12 relative: far below the 2e-3 output bar) and gets
//       8 channels x 4 tokens; the per-channel operands are the 4x8 transpose of that.
// Partials and the combine pass are those of the other decode kernels (decode_common.hpp).
#include "decode_common.hpp"

#include <algorithm>

namespace argus_decode {

namespace {

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef uint32_t u32_a2 __attribute__((aligned(2)));  // code words sit at 2-byte boundaries (18- and 34-byte blocks)

enum { kFmtQ4_0 = 0, kFmtQ4_1 = 1, kFmtQ8_0 = 2 };

template <int FMT>
struct BlockFmt {
  static constexpr int HDR = (FMT == kFmtQ4_1) ? 4 : 2;             // header bytes
  static constexpr int BB = HDR + ((FMT == kFmtQ8_0) ? 32 : 16);    // block bytes
  static constexpr int CW = (FMT == kFmtQ8_0) ? 2 : 1;              // code dwords per lane piece
};

// Element (within its block) held by slot s of the piece a lane with code index x loads.
template <int FMT>
__host__ __device__ constexpr int slot_elem(int x, int s) {
  return (FMT == kFmtQ8_0) ? 8 * x + s : (s < 4 ? 4 * x + s : 16 + 4 * x + (s - 4));
}

// What one lane holds of one block before it is dequantised.
template <int FMT>
struct RawPiece {
  uint32_t code[BlockFmt<FMT>::CW];
  uint32_t hdr;  // q4_0 / q8_0: f16 d in the low half; q4_1: f16 d | f16 m << 16
};

// The piece with code index x of the block at byte offset `blk` from `base` (`base` is wave-uniform
// and every offset is an unsigned 32-bit sum, so the load takes its address as base + lane offset).
template <int FMT>
__device__ __forceinline__ RawPiece<FMT> load_piece(const uint8_t *base, uint32_t blk, uint32_t x) {
  using F = BlockFmt<FMT>;
  RawPiece<FMT> p;
  if constexpr (FMT == kFmtQ4_1) p.hdr = *(const uint32_t *)(base + blk);
  else p.hdr = *(const uint16_t *)(base + blk);
#pragma unroll
  for (int w = 0; w < F::CW; ++w) p.code[w] = *(const u32_a2 *)(base + (blk + (uint32_t)F::HDR + 4u * ((uint32_t)F::CW * x + (uint32_t)w)));
  return p;
}

// Bytes b0 b1 b2 b3 of `bytes` (each < 256) -> halves {1024 + b0, 1024 + b1} and {1024 + b2, 1024 + b3}:
// 0x64 in the high byte of a half is the exponent of 1024, whose mantissa unit is 1.
__device__ __forceinline__ half2_t bytes_lo(uint32_t bytes) {
  return __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, bytes, 0x04010400u));
}
__device__ __forceinline__ half2_t bytes_hi(uint32_t bytes) {
  return __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, bytes, 0x04030402u));
}

// The 8 codes of a piece as exact f16 integers: n - 8 (q4_0), n (q4_1), c (q8_0).
template <int FMT>
__device__ __forceinline__ void piece_codes(const RawPiece<FMT> &p, half2_t (&v)[4]) {
  if constexpr (FMT == kFmtQ8_0) {
    // int8 c -> byte c + 128 -> 1024 + 128 + c
    const half2_t off = {(_Float16)-1152.0f, (_Float16)-1152.0f};
#pragma unroll
    for (int w = 0; w < 2; ++w) {
      const uint32_t u = p.code[w] ^ 0x80808080u;
      v[2 * w] = bytes_lo(u) + off;
      v[2 * w + 1] = bytes_hi(u) + off;
    }
  } else {
    const uint32_t lo = p.code[0] & 0x0f0f0f0fu, hi = (p.code[0] >> 4) & 0x0f0f0f0fu;
    const _Float16 o = (FMT == kFmtQ4_0) ? (_Float16)-1032.0f : (_Float16)-1024.0f;  // 1024 (and the zero point 8)
    const half2_t off = {o, o};
    v[0] = bytes_lo(lo) + off;
    v[1] = bytes_hi(lo) + off;
    v[2] = bytes_lo(hi) + off;
    v[3] = bytes_hi(hi) + off;
  }
}

template <int FMT>
__device__ __forceinline__ half8_t code_operand(const RawPiece<FMT> &p) {
  half2_t v[4];
  piece_codes<FMT>(p, v);
  return half8_t{v[0][0], v[0][1], v[1][0], v[1][1], v[2][0], v[2][1], v[3][0], v[3][1]};
}

// The 8 values of a piece, rounded once to f16: d * code (+ m).
template <int FMT>
__device__ __forceinline__ half8_t dequant_piece(const RawPiece<FMT> &p) {
  const half2_t dd = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0u, p.hdr, 0x01000100u));  // {d, d}
  half2_t v[4];
  piece_codes<FMT>(p, v);
  if constexpr (FMT == kFmtQ4_1) {
    const half2_t mm = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0u, p.hdr, 0x03020302u));  // {m, m}
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = __builtin_elementwise_fma(v[i], dd, mm);
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = v[i] * dd;
  }
  return half8_t{v[0][0], v[0][1], v[1][0], v[1][1], v[2][0], v[2][1], v[3][0], v[3][1]};
}

__device__ __forceinline__ float hdr_scale(uint32_t hdr) { return (float)__builtin_bit_cast(half2_t, hdr)[0]; }
__device__ __forceinline__ float hdr_min(uint32_t hdr) { return (float)__builtin_bit_cast(half2_t, hdr)[1]; }

// One element of a block as f32 (rare paths only).
template <int FMT>
__device__ float block_elem(const uint8_t *blk, int e) {
  using F = BlockFmt<FMT>;
  const float d = (float)*(const _Float16 *)blk;
  if constexpr (FMT == kFmtQ8_0) return d * (float)(int8_t)blk[F::HDR + e];
  const int byte = blk[F::HDR + (e & 15)];
  const int n = e < 16 ? (byte & 15) : (byte >> 4);
  if constexpr (FMT == kFmtQ4_0) return d * (float)(n - 8);
  return d * (float)n + (float)*(const _Float16 *)(blk + 2);
}

// Uniform-weights fallback of common.rs:806-813 for a block cache: out = mean of the attended V rows.
template <int FMT>
struct BlockFallback {
  static __device__ bool run(const DecodeParams &p, int b, int h, int D) {
    using F = BlockFmt<FMT>;
    const int kvh = h / p.group;
    const uint8_t *vb = (const uint8_t *)p.v + ((int64_t)b * p.kv_bs + (int64_t)kvh * p.head_stride) / 32 * F::BB;
    const float u = 1.0f / (float)p.len;
    for (int c = threadIdx.x; c < D; c += blockDim.x) {
      float acc = 0.0f;
      for (int t = 0; t < p.len; ++t)
        acc += u * block_elem<FMT>(vb + ((int64_t)(p.kv_start + t) * p.row_stride / 32 + c / 32) * F::BB, c % 32);
      p.out[(int64_t)b * p.out_bs + (int64_t)h * D + c] = acc;
    }
    if (p.scores) {
      float *srow = p.scores + (int64_t)b * p.score_bs + (int64_t)h * p.score_stride;
      for (int t = threadIdx.x; t < p.len; t += blockDim.x) srow[t] = u;
    }
    return true;
  }
};

constexpr int kWaves = 4;

template <int D>
struct BlockShape {
  static constexpr int KK = D / 32;                       // blocks per row
  static constexpr int VSEG = (D + 127) / 128;            // V pieces per lane per row (8 channels each)
  static constexpr int NACC = 8 * VSEG;                   // O accumulators (float4 each)
  static constexpr int MAXH = (D == 256) ? 8 : 16;        // query heads per KV head (bounds the merge LDS)
};

template <int FMT, int D, int TW>
__global__ __launch_bounds__(64 * kWaves) void decode_blocks_kernel(const DecodeParams p) {
  using F = BlockFmt<FMT>;
  using SH = BlockShape<D>;
  constexpr int KK = SH::KK, VSEG = SH::VSEG, NACC = SH::NACC;
  constexpr int TILE = 16 * TW;  // tokens per wave iteration
  constexpr float kLn2 = 0.6931471805599453f;

  const int split = blockIdx.x, kvh = blockIdx.y, b = blockIdx.z;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int j = lane >> 4, r = lane & 15;
  const int G = p.group;

  const int t_begin = split * p.chunk;
  const int t_end = min(p.len, t_begin + p.chunk);

  // Strides arrive in elements; rows are whole blocks.  Within one head's slab everything is
  // addressed by a 32-bit byte offset (checked by the launcher) built with 24-bit multiplies.
  const uint32_t row_bytes = (uint32_t)(p.row_stride / 32 * F::BB);
  const int64_t head_off = ((int64_t)b * p.kv_bs + (int64_t)kvh * p.head_stride) / 32 * F::BB + (int64_t)p.kv_start * row_bytes;
  const uint8_t *kb = (const uint8_t *)p.k + head_off;
  const uint8_t *vb = (const uint8_t *)p.v + head_off;
  // V piece sg of a lane: block vblk[sg], code index r % 4 (head_dim 64 has two blocks: lanes 8..15 repeat 0..7)
  int vblk[VSEG];
#pragma unroll
  for (int sg = 0; sg < VSEG; ++sg) vblk[sg] = (4 * sg + r / 4) % KK;

  RawPiece<FMT> kraw[TW][KK];
  RawPiece<FMT> vraw[TW][VSEG][4];
  // Rows past the chunk re-read its last row (they are masked below), so every request is
  // unconditional and a tile may be asked for before it is known to exist.
  const int last = t_end - 1;
  auto load_k = [&](int base) {
#pragma unroll
    for (int tw = 0; tw < TW; ++tw) {
      const uint32_t off = __umul24((uint32_t)min(base + 16 * tw + r, last), row_bytes);
#pragma unroll
      for (int kk = 0; kk < KK; ++kk) kraw[tw][kk] = load_piece<FMT>(kb, off + (uint32_t)(kk * F::BB), (uint32_t)j);
    }
  };
  auto load_v = [&](int base) {
#pragma unroll
    for (int tw = 0; tw < TW; ++tw)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const uint32_t off = __umul24((uint32_t)min(base + 16 * tw + 4 * j + e, last), row_bytes);
#pragma unroll
        for (int sg = 0; sg < VSEG; ++sg) vraw[tw][sg][e] = load_piece<FMT>(vb, off + (uint32_t)(vblk[sg] * F::BB), (uint32_t)(r & 3));
      }
  };
  const int base0 = t_begin + __builtin_amdgcn_readfirstlane(wave) * TILE;
  load_k(base0);
  load_v(base0);
  __builtin_amdgcn_sched_barrier(0);  // keep these requests ahead of the query's

  // ---- Q operand: lane (j, h = r), block kk: the elements slot_elem(j, 0..7), log2 domain, hi + lo
  half8_t qh[KK], ql[KK];
  float qsum[KK];  // q4_1 only: sum of the scaled query over block kk, for the m term
  {
    const float c = p.scale * 1.4426950408889634f;
    const int h = kvh * G + min(r, G - 1);
    const float *qp = p.q + (int64_t)b * p.q_bs + (int64_t)h * D;
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
      float qv[8];
#pragma unroll
      for (int s = 0; s < 8; ++s) qv[s] = qp[32 * kk + slot_elem<FMT>(j, s)];  // lanes past the group re-read its last head
      loaded8(qv);
      float part = 0.0f;
#pragma unroll
      for (int s = 0; s < 8; ++s) {
        const float x = (r < G) ? qv[s] * c : 0.0f;
        part += x;
        _Float16 hi, lo;
        split_f16(x, hi, lo);
        qh[kk][s] = hi;
        ql[kk][s] = lo;
      }
      // the four lane groups hold the four quarters of the block
      part += __shfl_xor(part, 16, 64);
      part += __shfl_xor(part, 32, 64);
      qsum[kk] = part;
    }
  }
  // Result lane (j, h) of a logits MFMA holds tokens 4j..4j+3; their block headers were loaded by
  // lanes 16j + (4j + i) (token = lane % 16).
  int hdr_src[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) hdr_src[i] = 4 * (20 * j + i);  // ds_bpermute byte address

  float4_t o_acc[NACC];
#pragma unroll
  for (int a = 0; a < NACC; ++a) o_acc[a] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
  float m_run = kNegInf, l_run = 0.0f;  // per (lane = head r); l is this lane group's partial sum

  for (int base = base0; base < t_end; base += kWaves * TILE) {
    // ---- logits ---------------------------------------------------------------------------------
    float4_t s[TW];
#pragma unroll
    for (int tw = 0; tw < TW; ++tw) {
      s[tw] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
      for (int kk = 0; kk < KK; ++kk) {
        const half8_t ka = code_operand<FMT>(kraw[tw][kk]);
        float4_t dot = {0.0f, 0.0f, 0.0f, 0.0f};
        dot = __builtin_amdgcn_mfma_f32_16x16x32_f16(ka, qh[kk], dot, 0, 0, 0);
        dot = __builtin_amdgcn_mfma_f32_16x16x32_f16(ka, ql[kk], dot, 0, 0, 0);
        const int d_own = __builtin_bit_cast(int, hdr_scale(kraw[tw][kk].hdr));
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float d_tok = __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(hdr_src[i], d_own));
          s[tw][i] = fmaf(d_tok, dot[i], s[tw][i]);
        }
        if constexpr (FMT == kFmtQ4_1) {
          const int m_own = __builtin_bit_cast(int, hdr_min(kraw[tw][kk].hdr));
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const float m_tok = __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(hdr_src[i], m_own));
            s[tw][i] = fmaf(m_tok, qsum[kk], s[tw][i]);
          }
        }
      }
    }
    load_k(base + kWaves * TILE);  // the K registers are free again: request the wave's next tile
    const bool full = base + TILE <= t_end;
    float mt = kNegInf;
#pragma unroll
    for (int tw = 0; tw < TW; ++tw)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float sv = fmaxf(s[tw][i], kNegInf);  // NaN logit counts as -inf (common.rs:790-795)
        if (!full && base + 16 * tw + 4 * j + i >= t_end) sv = kNegInf;
        s[tw][i] = sv;
        mt = fmaxf(mt, sv);
      }
    if (p.scores && r < G) {
      // Logits in natural units; the combine pass rewrites them as probabilities.
      float *srow = p.scores + (int64_t)b * p.score_bs + (int64_t)(kvh * G + r) * p.score_stride;
#pragma unroll
      for (int tw = 0; tw < TW; ++tw)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int t = base + 16 * tw + 4 * j + i;
          if (t < t_end) srow[t] = s[tw][i] * kLn2;
        }
    }

    // ---- online softmax: the running max of a head is shared by the four lane groups -----------
    mt = fmaxf(mt, __shfl_xor(mt, 16, 64));
    mt = fmaxf(mt, __shfl_xor(mt, 32, 64));
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
        // The row sum takes the unrounded weight: it also normalises the emitted scores, and over
        // a handful of tokens the f16 roundings of the weights (2^-12 each) would not average out.
        const float e = __builtin_amdgcn_exp2f(s[tw][i] - m_ref);
        lsum += e;
        pa[tw][i] = (_Float16)e;
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
      for (int sg = 0; sg < VSEG; ++sg) {
        half8_t vrow[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) vrow[e] = dequant_piece<FMT>(vraw[tw][sg][e]);
#pragma unroll
        for (int c = 0; c < 8; ++c) {
          const half4_t bv = {vrow[0][c], vrow[1][c], vrow[2][c], vrow[3][c]};
          o_acc[sg * 8 + c] = __builtin_amdgcn_mfma_f32_16x16x16f16(pa[tw], bv, o_acc[sg * 8 + c], 0, 0, 0);
        }
      }
    load_v(base + kWaves * TILE);
  }

  // ---- merge: lane groups (row sum), then the waves through LDS ---------------------------------
  l_run += __shfl_xor(l_run, 16, 64);
  l_run += __shfl_xor(l_run, 32, 64);
  __shared__ float lds_m[kWaves][16], lds_l[kWaves][16];
  __shared__ float lds_acc[kWaves][SH::MAXH][D + 4];
  if (j == 0) {
    lds_m[wave][r] = m_run;
    lds_l[wave][r] = l_run;
  }
  if (r < 4 * KK || VSEG > 1) {  // head_dim 64: lanes 8..15 hold copies
#pragma unroll
    for (int sg = 0; sg < VSEG; ++sg)
#pragma unroll
      for (int c = 0; c < 8; ++c)
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (4 * j + i < SH::MAXH) lds_acc[wave][4 * j + i][32 * vblk[sg] + slot_elem<FMT>(r & 3, c)] = o_acc[sg * 8 + c][i];
  }
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
    // Partials are handed to the combine pass in natural-log units.
    const int64_t pidx = ((int64_t)b * p.n_heads_q + h) * p.nsplit + split;
    p.ws_o[pidx * D + c] = o;
    if (c == 0) {
      p.ws_ml[pidx * 2 + 0] = mm * kLn2;
      p.ws_ml[pidx * 2 + 1] = ll;
    }
  }
}

template <int FMT, int D>
int launch_blocks(argus_hip_ctx *ctx, DecodeParams &p, int batch, hipStream_t stream) {
  constexpr int TW = 2;
  constexpr int tile_rows = kWaves * 16 * TW;
  static int wgs_per_cu = 0;  // per instantiation; single inference thread
  if (wgs_per_cu == 0) {
    int n = 0;
    ARGUS_HIP_CHECK(ctx, hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, decode_blocks_kernel<FMT, D, TW>, 64 * kWaves, 0));
    wgs_per_cu = std::max(1, n);
  }
  choose_splits(p, batch * p.n_heads_kv, tile_rows, (int64_t)ctx->compute_units * wgs_per_cu);
  p.direct = 0;
  const size_t n_part = (size_t)batch * p.n_heads_q * p.nsplit;
  const size_t ml_bytes = (n_part * 2 * sizeof(float) + 255) / 256 * 256;
  int rc = argus_ws_reserve(ctx, ml_bytes + n_part * D * sizeof(float));
  if (rc != ARGUS_HIP_OK) return rc;
  p.ws_ml = ctx->ws;
  p.ws_o = (float *)((char *)ctx->ws + ml_bytes);
  {
    KernelTimer timer(ctx, stream);
    hipLaunchKernelGGL((decode_blocks_kernel<FMT, D, TW>), dim3(p.nsplit, p.n_heads_kv, batch), dim3(64 * kWaves), 0, stream, p);
  }
  ARGUS_HIP_CHECK(ctx, hipGetLastError());
  hipLaunchKernelGGL((decode_combine_kernel<BlockFallback<FMT>, D>), dim3(p.n_heads_q, batch), dim3(256), 0, stream, p);
  ARGUS_HIP_CHECK(ctx, hipGetLastError());
  return ARGUS_HIP_OK;
}

template <int FMT>
int launch_blocks_dim(argus_hip_ctx *ctx, DecodeParams &p, int D, int batch, hipStream_t stream) {
  switch (D) {
    case 64: return launch_blocks<FMT, 64>(ctx, p, batch, stream);
    case 128: return launch_blocks<FMT, 128>(ctx, p, batch, stream);
    default: return launch_blocks<FMT, 256>(ctx, p, batch, stream);
  }
}

}  // namespace

int launch_decode_blocks(argus_hip_ctx *ctx, DecodeParams &p, int D, int kv_dtype, int batch, hipStream_t stream) {
  if (p.kv_index || p.softcap > 0.0f)
    return argus_fail(ctx, ARGUS_HIP_ERR_UNSUPPORTED,
                      "attention_gen: block-quantised caches take no index list or soft-cap; decode them with "
                      "argus_hip_kv_decode_descriptor and attend the F16 copy");
  if (p.group > ((D == 256) ? 8 : 16))
    return argus_fail(ctx, ARGUS_HIP_ERR_UNSUPPORTED, "attention_gen: %d query heads per KV head on a block-quantised cache", p.group);
  if ((p.row_stride % 32) || (p.head_stride % 32) || (p.kv_bs % 32))
    return argus_fail(ctx, ARGUS_HIP_ERR_INVALID, "attention_gen: block-quantised cache strides must be whole 32-element blocks");
  // rows are addressed as (row index, 24 bits) x (row bytes, 24 bits) -> 32-bit byte offset
  if (p.len >= (1 << 24) || p.row_stride / 32 * 34 >= (1 << 24) || (int64_t)p.len * (p.row_stride / 32 * 34) > 0xffffffffll)
    return argus_fail(ctx, ARGUS_HIP_ERR_UNSUPPORTED, "attention_gen: block-quantised head slab beyond 4 GiB");
  switch (kv_dtype) {
    case ARGUS_HIP_Q4_0: return launch_blocks_dim<kFmtQ4_0>(ctx, p, D, batch, stream);
    case ARGUS_HIP_Q4_1: return launch_blocks_dim<kFmtQ4_1>(ctx, p, D, batch, stream);
    default: return launch_blocks_dim<kFmtQ8_0>(ctx, p, D, batch, stream);
  }
}

}  // namespace argus_decode
