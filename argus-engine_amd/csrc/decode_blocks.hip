// Split-KV flash-decode over block-quantised caches (q4_0, q4_1, q8_0, q2_0), dequantised in registers.
//
// The Q4_0 arm of Backend::attention_gen (engine/src/backend/cpu/common.rs:676-850: dequantise each
// K / V row, then the F32 algorithm with its NaN and uniform-weights guards) and the in-kernel form
// of the `--kv-format` attention whose reference floor decodes the whole cache to F32 first
// (engine/src/kv/standard_format.rs:538-643).  Blocks are the descriptor formats of
// engine/src/format/dtype_layout.rs:102-166 with 32 elements: [f16 d][f16 m?][codes];
// q4_0: x = d * (n - 8), q4_1: x = d * n + m, n = 4-bit code, element i in the low nibble of code
// byte i, element 16 + i in the high nibble; q8_0: x = d * c, c = int8; q2_0: [f16 d][f16 m][8 code
// bytes], x = d * n + m, element 4i + k in bits 2k, 2k+1 of code byte i (dtype_layout.rs:146-166).
//
// Same data flow as decode_mfma.hip.  Packed rows read without an index list are streamed: a wave
// fetches its tile as one contiguous run, parks it in a private LDS copy and every lane reads the
// pieces of its operands from there (STREAM, see the kernel).  Otherwise rows are requested one
// whole block per lane (contiguous 16 or 32 code bytes, so a request touches each cache line once)
// and the lanes then trade dwords (v_permlane swaps for K, a wave-private LDS strip for 4-bit V
// rows).  Either way each lane ends up with the 4 (q4) or 8 (q8) code bytes of its MFMA operand,
// which it turns into 8 f16 values: q8 bytes go under the exponent of 1024 with v_perm and a packed
// subtract leaves the exact integer; q4 nibbles are masked into the mantissa of 64 + n.
//   S^T[token][head] = sum over blocks kk of d_kk(token) * (C_kk . Q_kk^T)
//       v_mfma_f32_16x16x32_f16 per 32-element block with A = the integer codes n - 8 (q4_0), n
//       (q4_1) or c (q8_0) -- lane (j, r) = token r, code bytes 4j..4j+3 of block kk, i.e. elements
//       {4j..4j+3, 16+4j..16+4j+3} (q8: elements 8j..8j+7) -- and B = the same elements of Q as
//       f16 hi + lo, so the block dot products are exact to f32.  The scale is applied to the MFMA
//       result: the result lane (j, h) holds tokens 4j..4j+3, whose scales sit in lanes 20j + i of
//       the wave and are fetched with ds_bpermute (q4_1 adds m_kk(token) * sum of Q_kk).  Logits
//       therefore carry no f16 rounding of d * (n - 8), and the emitted scores keep the 1e-4 bar.
//       With at most four query heads per KV head (eight at head_dim 64, and at 128 when no scores
//       are emitted) the two operands change places (TOKCOL, see the kernel): S[head][token], the
//       result lane (j, n) holds token n, lane group j keeps head j (heads 2j, 2j + 1) and applies
//       the scales of its own token; the query's hi and lo parts are two rows of the one operand.
//   O[head][channel] = P . V     v_mfma_f32_16x16x16_f16 (16x16x32 over two tiles at head_dim 128, TOKCOL)
//       B: lane (j, r) loads, for tokens 4j..4j+3, code bytes 4(r%4).. of block r/4, dequantises
//       them to f16 (one rounding, 2^-12 relative: far below the 2e-3 output bar) and gets
//       8 channels x 4 tokens; the per-channel operands are the 4x8 transpose of that.
//       TOKCOL: the V operand is the bare code and the block scale multiplies the P operand instead,
//       whose spare rows hold one copy of the weights per block of output columns.
// Partials and the combine pass are those of the other decode kernels (decode_common.hpp).
#include "decode_common.hpp"

#include <algorithm>

namespace argus_decode {

namespace {

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
// LDS as 32-bit addresses (the streamed tile copies are read through lane bases kept as integers)
typedef const __attribute__((address_space(3))) uint32_t *lds_u32_ptr;
typedef const __attribute__((address_space(3))) uint16_t *lds_u16_ptr;
__device__ __forceinline__ uint32_t lds_address(const void *p) {
  return (uint32_t)(uintptr_t)(const __attribute__((address_space(3))) void *)p;
}
__device__ __forceinline__ uint32_t lds_dword(uint32_t addr) { return *(lds_u32_ptr)(uintptr_t)addr; }
__device__ __forceinline__ uint32_t lds_half(uint32_t addr) { return *(lds_u16_ptr)(uintptr_t)addr; }
typedef uint32_t u32_a2 __attribute__((aligned(2)));  // code words sit at 2-byte boundaries (18- and 34-byte blocks)

enum { kFmtQ4_0 = 0, kFmtQ4_1 = 1, kFmtQ8_0 = 2, kFmtQ2_0 = 3 };
constexpr int kBufferFlags = 0x00020000;  // raw buffer, bounds-checked against num_records

// Orders a wave's LDS accesses for the compiler when its lanes exchange data through LDS.
__device__ __forceinline__ void wave_lds_fence() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

template <int FMT>
struct BlockFmt {
  static constexpr bool kHasMin = FMT == kFmtQ4_1 || FMT == kFmtQ2_0;  // header is (d, m)
  static constexpr int HDR = kHasMin ? 4 : 2;                                          // header bytes
  static constexpr int CODE_DW = (FMT == kFmtQ8_0) ? 8 : ((FMT == kFmtQ2_0) ? 2 : 4);  // code dwords per block
  static constexpr int BB = HDR + 4 * CODE_DW;                                         // block bytes
  // code dwords per lane piece (q2_0: the piece is one 16-bit half of its dword)
  static constexpr int CW = (FMT == kFmtQ8_0) ? 2 : 1;
};

// Element (within its block) held by slot s of the piece a lane with code index x loads
// (q4: the slots follow the order in which the shifts below bring the nibbles out).
template <int FMT>
__host__ __device__ constexpr int slot_elem(int x, int s) {
  if (FMT == kFmtQ8_0) return 8 * x + s;
  if (FMT == kFmtQ2_0) return 8 * x + (s >> 1) + 4 * (s & 1);  // slot 2f + h: field f of byte 2x + h
  const int within = (s & 3) == 1 ? 2 : ((s & 3) == 2 ? 1 : (s & 3));  // 0, 2, 1, 3
  return (s < 4 ? 0 : 16) + 4 * x + within;
}

// How the operands carry a code.  q4: the nibble n sits in mantissa bits 4..7 (where the high
// nibble of a byte already is) under the exponent of 64, i.e. the half is exactly 64 + n, with no
// arithmetic at all; the bias (and q4_0's zero point 8) is taken out where it is cheap: from the
// block dot product as (bias + zero) * sum(Q), folded into the accumulator the MFMA starts from,
// and from the values as one fma whose addend -64 d is exact.  q8: the int8 c is made exact by a
// packed subtract (bias 0).
// q2_0 (x = d * n + m, four 2-bit codes per byte, element 4i + k in bits 2k.. of byte i) works the
// same way with two positions: fields 0 and 1 are shifted up by 4, so every code sits at bits 4..5
// (under the exponent of 64) or bits 6..7 (under the exponent of 16) and the bias depends on the slot.
template <int FMT>
struct Codec {
  static constexpr float kBias = (FMT == kFmtQ8_0) ? 0.0f : 64.0f;  // operand = kBias + code (q2_0: slot_bias)
  static constexpr float kZero = (FMT == kFmtQ4_0) ? 8.0f : 0.0f;   // value = d * (code - kZero) (+ m)
  static __host__ __device__ constexpr float slot_bias(int s) {
    return (FMT == kFmtQ2_0) ? (((s >> 1) & 1) ? 16.0f : 64.0f) : kBias;
  }
};

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
  if constexpr (F::kHasMin) p.hdr = *(const uint32_t *)(base + blk);
  else p.hdr = *(const uint16_t *)(base + blk);
#pragma unroll
  for (int w = 0; w < F::CW; ++w) p.code[w] = *(const u32_a2 *)(base + (blk + (uint32_t)F::HDR + 4u * ((uint32_t)F::CW * x + (uint32_t)w)));
  return p;
}

// A whole block as one lane loads it: the rows of a tile are read one block per lane (16 or 32
// contiguous code bytes), which touches each cache line of the tile once per request instead of
// once per 4-byte piece, and the lanes then trade dwords (block_to_pieces, the V strip).
template <int FMT>
struct RawBlock {
  uint32_t code[BlockFmt<FMT>::CODE_DW];
  uint32_t hdr;
};
typedef uint32_t u32x4_a2 __attribute__((ext_vector_type(4), aligned(2)));

template <int FMT>
__device__ __forceinline__ RawBlock<FMT> load_block(const uint8_t *base, uint32_t blk) {
  using F = BlockFmt<FMT>;
  RawBlock<FMT> b;
  if constexpr (F::kHasMin) b.hdr = *(const uint32_t *)(base + blk);
  else b.hdr = *(const uint16_t *)(base + blk);
  if constexpr (FMT == kFmtQ2_0) {
    typedef uint32_t u32x2_a4 __attribute__((ext_vector_type(2), aligned(4)));
    const u32x2_a4 c = *(const u32x2_a4 *)(base + (blk + (uint32_t)F::HDR));
    b.code[0] = c[0];
    b.code[1] = c[1];
  } else {
#pragma unroll
    for (int w = 0; w < F::CW; ++w) {
      const u32x4_a2 c = *(const u32x4_a2 *)(base + (blk + (uint32_t)F::HDR + 16u * (uint32_t)w));
#pragma unroll
      for (int i = 0; i < 4; ++i) b.code[4 * w + i] = c[i];
    }
  }
  return b;
}

// v_permlane16_swap / v_permlane32_swap: trade the odd rows, or the upper half, of the first register
// with the even rows, or the lower half, of the second.
struct SwapPair {
  uint32_t first, second;
};
__device__ __forceinline__ SwapPair permlane16_swap(uint32_t a, uint32_t b) {
  const auto r = __builtin_amdgcn_permlane16_swap(a, b, false, false);
  return {r[0], r[1]};
}
__device__ __forceinline__ SwapPair permlane32_swap(uint32_t a, uint32_t b) {
  const auto r = __builtin_amdgcn_permlane32_swap(a, b, false, false);
  return {r[0], r[1]};
}

// 4 x 4 transpose across the four lane groups (lanes 16 apart): lane group j ends up with what lane
// groups 0..3 held in v[j]: the 16-lane swap trades v[0], v[2] of the odd groups with v[1], v[3]
// of the even ones, the 32-lane swap does the same between the halves of the wave.
__device__ __forceinline__ void transpose_lane_groups(uint32_t (&v)[4]) {
  const SwapPair a = permlane16_swap(v[0], v[1]);
  const SwapPair b = permlane16_swap(v[2], v[3]);
  const SwapPair c = permlane32_swap(a.first, b.first);
  const SwapPair d = permlane32_swap(a.second, b.second);
  v[0] = c.first; v[2] = c.second; v[1] = d.first; v[3] = d.second;
}

// Lane group j holds block j of its row; afterwards piece[kk] is the lane's piece (code index j)
// of block kk, with that block's header.
template <int FMT>
__device__ __forceinline__ void block_to_pieces(const RawBlock<FMT> &b, RawPiece<FMT> (&piece)[4]) {
  constexpr int CW = BlockFmt<FMT>::CW;
#pragma unroll
  for (int w = 0; w < CW; ++w) {
    // piece dword w of code index x is block dword CW * x + w
    uint32_t v[4];
#pragma unroll
    for (int x = 0; x < 4; ++x) {
      if constexpr (FMT == kFmtQ2_0) v[x] = b.code[x >> 1];  // the dword that holds half x
      else v[x] = b.code[CW * x + w];
    }
    transpose_lane_groups(v);
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) piece[kk].code[w] = v[kk];
  }
  // headers: all-gather over the lane groups with the same two trades
  const SwapPair p = permlane16_swap(b.hdr, b.hdr);        // (even group's, odd group's)
  const SwapPair lo = permlane32_swap(p.first, p.first);   // (group 0's, group 2's)
  const SwapPair hi = permlane32_swap(p.second, p.second); // (group 1's, group 3's)
  piece[0].hdr = lo.first; piece[2].hdr = lo.second; piece[1].hdr = hi.first; piece[3].hdr = hi.second;
}

// Bytes b0 b1 b2 b3 of `bytes` (each < 256) -> halves {1024 + b0, 1024 + b1} and {1024 + b2, 1024 + b3}:
// 0x64 in the high byte of a half is the exponent of 1024, whose mantissa unit is 1.
__device__ __forceinline__ half2_t bytes_lo(uint32_t bytes) {
  return __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, bytes, 0x04010400u));
}
__device__ __forceinline__ half2_t bytes_hi(uint32_t bytes) {
  return __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, bytes, 0x04030402u));
}
// Two nibbles of a code word, 16 bits apart and already at bits 4..7 / 20..23 -> {64 + n, 64 + n'}.
// One v_and_or_b32 when the callers keep `mask` and `exponent` in vector registers (this target's
// three-operand form takes no literal).  Plain C on purpose: an instruction written as inline asm is
// invisible to the compiler's hazard recogniser, and a VALU write into a register that an MFMA in
// flight still reads as its accumulator input needs wait states that only the recogniser inserts.
// Spelled as asm, this function overwrote such registers in some builds (wrong logits for q4_1 and
// q2_0, depending on what the scheduler placed behind the MFMAs).
__device__ __forceinline__ half2_t nibbles(uint32_t word, uint32_t mask, uint32_t exponent) {
  return __builtin_bit_cast(half2_t, (word & mask) | exponent);
}

// v_perm selector that spreads one 16-bit half of a dword as [byte, 0, next byte, 0] (q2_0 pieces).
__device__ __forceinline__ uint32_t q2_half_selector(int half) { return half ? 0x0c030c02u : 0x0c010c00u; }

// The 8 codes of a piece as exact f16 numbers Codec::slot_bias + code.  `sel` (q2_0 only): the
// lane's q2_half_selector.
template <int FMT>
__device__ __forceinline__ void piece_codes(const RawPiece<FMT> &p, half2_t (&v)[4], uint32_t sel) {
  if constexpr (FMT == kFmtQ2_0) {
    const uint32_t w = __builtin_amdgcn_perm(0u, p.code[0], sel);  // [byte 2x, 0, byte 2x+1, 0]
    const uint32_t w4 = w << 4;
    uint32_t mask_a = 0x00300030u, exp_a = 0x54005400u, mask_b = 0x00c000c0u, exp_b = 0x4c004c00u;
    asm("" : "+v"(mask_a), "+v"(exp_a), "+v"(mask_b), "+v"(exp_b));
    v[0] = nibbles(w4, mask_a, exp_a);  // field 0 -> bits 4..5: 64 + n
    v[1] = nibbles(w4, mask_b, exp_b);  // field 1 -> bits 6..7: 16 + n
    v[2] = nibbles(w, mask_a, exp_a);   // field 2
    v[3] = nibbles(w, mask_b, exp_b);   // field 3
  } else if constexpr (FMT == kFmtQ8_0) {
    // int8 c -> byte c + 128 -> 1024 + 128 + c
    const half2_t off = {(_Float16)-1152.0f, (_Float16)-1152.0f};
#pragma unroll
    for (int w = 0; w < 2; ++w) {
      const uint32_t u = p.code[w] ^ 0x80808080u;
      v[2 * w] = bytes_lo(u) + off;
      v[2 * w + 1] = bytes_hi(u) + off;
    }
  } else {
    const uint32_t w = p.code[0];
    uint32_t mask = 0x00f000f0u, exponent = 0x54005400u;
    asm("" : "+v"(mask), "+v"(exponent));  // keep both in vector registers
    v[0] = nibbles(w << 4, mask, exponent);  // low nibbles of bytes 0, 2
    v[1] = nibbles(w >> 4, mask, exponent);  // low nibbles of bytes 1, 3
    v[2] = nibbles(w, mask, exponent);       // high nibbles of bytes 0, 2
    v[3] = nibbles(w >> 8, mask, exponent);  // high nibbles of bytes 1, 3
  }
}

template <int FMT>
__device__ __forceinline__ half8_t code_operand(const RawPiece<FMT> &p, uint32_t sel) {
  half2_t v[4];
  piece_codes<FMT>(p, v, sel);
  return half8_t{v[0][0], v[0][1], v[1][0], v[1][1], v[2][0], v[2][1], v[3][0], v[3][1]};
}

// The values d * code of the pieces of two tokens (4-bit formats), slot by slot: out[s] = {token a's
// value of slot s, token b's}.  The code words are interleaved first -- bytes 0, 1 of both tokens in
// one word, bytes 2, 3 in another -- and the four shifts of piece_codes then bring out one nibble
// position of both tokens at a time: byte 0 low, byte 1 low, byte 0 high, byte 1 high from the first
// word are slots 0, 2, 4, 6, the same from the second word slots 1, 3, 5, 7.
// SCALED = false leaves the operands 64 + code (the caller scales the other MFMA operand instead).
template <int FMT, int N, bool SCALED>
__device__ __forceinline__ void scaled_pair(const RawPiece<FMT> &a, const RawPiece<FMT> &b, uint32_t upper, half2_t (&out)[N]) {
  static_assert((FMT == kFmtQ4_0 || FMT == kFmtQ4_1) && (N == 8 || N == 4), "nibble formats; whole or half pieces");
  half2_t dd = {}, nb = {};
  if constexpr (SCALED) {
    dd = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(b.hdr, a.hdr, 0x05040100u));  // {d_a, d_b}
    nb = dd * half2_t{(_Float16)-64.0f, (_Float16)-64.0f};                               // exact
  }
  auto value = [&](half2_t code) { return SCALED ? __builtin_elementwise_fma(code, dd, nb) : code; };
  uint32_t mask = 0x00f000f0u, exponent = 0x54005400u;
  asm("" : "+v"(mask), "+v"(exponent));  // keep both in vector registers
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    uint32_t w = __builtin_amdgcn_perm(b.code[0], a.code[0], h ? 0x07060302u : 0x05040100u);
    if constexpr (N == 4) {
      // Half pieces (head_dim 64): the lane's half is the low or the high nibbles (`upper`); a
      // per-lane shift brings byte 0's to bits 4..7, and byte 1's follow 8 bits further up.  Slots
      // 0..3 are bytes 0, 2, 1, 3 of that half.
      w <<= 4u - 4u * upper;
      out[0 + h] = value(nibbles(w, mask, exponent));
      out[2 + h] = value(nibbles(w >> 8, mask, exponent));
    } else {
      out[0 + h] = value(nibbles(w << 4, mask, exponent));
      out[2 + h] = value(nibbles(w >> 4, mask, exponent));
      out[4 + h] = value(nibbles(w, mask, exponent));
      out[6 + h] = value(nibbles(w >> 8, mask, exponent));
    }
  }
}

// The same for q2_0 (four 2-bit fields per byte): byte h of both tokens' pieces goes into one word
// as [byte of a, 0, byte of b, 0] (`sel[h]`: the lane's v_perm selectors over {a's code dword, b's}),
// and the two masks of piece_codes bring out one field of both tokens at a time: field f of byte h
// is slot 2f + h of a whole piece (N = 8, two bytes) or slot f of a half piece (N = 4, one byte,
// sel[0]).  Values are d * code (SCALED) or the operands slot bias + code.
template <int N, bool SCALED>
__device__ __forceinline__ void scaled_pair_q2(const RawPiece<kFmtQ2_0> &a, const RawPiece<kFmtQ2_0> &b, const uint32_t (&sel)[2], half2_t (&out)[N]) {
  static_assert(N == 8 || N == 4, "whole or half pieces");
  half2_t dd = {}, nb_a = {}, nb_b = {};
  if constexpr (SCALED) {
    dd = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(b.hdr, a.hdr, 0x05040100u));  // {d_a, d_b}
    nb_a = dd * half2_t{(_Float16)-64.0f, (_Float16)-64.0f};                            // exact
    nb_b = dd * half2_t{(_Float16)-16.0f, (_Float16)-16.0f};
  }
  uint32_t mask_a = 0x00300030u, exp_a = 0x54005400u, mask_b = 0x00c000c0u, exp_b = 0x4c004c00u;
  asm("" : "+v"(mask_a), "+v"(exp_a), "+v"(mask_b), "+v"(exp_b));
  auto value = [&](half2_t code, half2_t nb) { return SCALED ? __builtin_elementwise_fma(code, dd, nb) : code; };
  constexpr int NB = N / 4;  // bytes of the piece
#pragma unroll
  for (int h = 0; h < NB; ++h) {
    const uint32_t w = __builtin_amdgcn_perm(b.code[0], a.code[0], sel[h]), w4 = w << 4;
    out[0 * NB + h] = value(nibbles(w4, mask_a, exp_a), nb_a);  // field 0 -> bits 4..5: 64 + n
    out[1 * NB + h] = value(nibbles(w4, mask_b, exp_b), nb_b);  // field 1 -> bits 6..7: 16 + n
    out[2 * NB + h] = value(nibbles(w, mask_a, exp_a), nb_a);   // field 2
    out[3 * NB + h] = value(nibbles(w, mask_b, exp_b), nb_b);   // field 3
  }
}

// The same for q8_0: bytes 0, 1 (2, 3) of both tokens' code words go into one word as [a's, b's,
// a's, b's], and the two byte spreads of piece_codes then yield one channel of both tokens each.
// N = 8: two code words per token; N = 4 (head_dim 64): the half piece's one word.
template <int N, bool SCALED>
__device__ __forceinline__ void scaled_pair_q8(const RawPiece<kFmtQ8_0> &a, const RawPiece<kFmtQ8_0> &b, half2_t (&out)[N]) {
  static_assert(N == 8 || N == 4, "whole or half pieces");
  const half2_t off = {(_Float16)-1152.0f, (_Float16)-1152.0f};
  half2_t dd = {};
  if constexpr (SCALED) dd = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(b.hdr, a.hdr, 0x05040100u));  // {d_a, d_b}
#pragma unroll
  for (int w = 0; w < N / 4; ++w)
#pragma unroll
    for (int k = 0; k < 2; ++k) {
      const uint32_t u = __builtin_amdgcn_perm(b.code[w], a.code[w], k ? 0x07030602u : 0x05010400u) ^ 0x80808080u;
      half2_t lo = bytes_lo(u) + off, hi = bytes_hi(u) + off;
      if constexpr (SCALED) {
        lo = lo * dd;
        hi = hi * dd;
      }
      out[4 * w + 2 * k] = lo;
      out[4 * w + 2 * k + 1] = hi;
    }
}

// Half a piece (head_dim 64, where 8 lanes would cover the two blocks of a row twice over): the
// element held by slot s of the half `upper` of code index x.  q4: `upper` selects the high nibbles;
// q8: the piece's second code word; q2_0: its second byte.
template <int FMT>
__host__ __device__ constexpr int half_slot_elem(int x, int upper, int s) {
  if (FMT == kFmtQ8_0 || FMT == kFmtQ2_0) return 8 * x + 4 * upper + s;
  return 16 * upper + 4 * x + (s == 1 ? 2 : (s == 2 ? 1 : s));  // 0, 2, 1, 3
}
// The operand of half slot s is half_slot_bias(s) + code.
template <int FMT>
__host__ __device__ constexpr float half_slot_bias(int s) {
  return (FMT == kFmtQ8_0) ? 0.0f : ((FMT == kFmtQ2_0 && (s & 1)) ? 16.0f : 64.0f);
}
// One element of a block as f32 (rare paths only).
template <int FMT>
__device__ float block_elem(const uint8_t *blk, int e) {
  using F = BlockFmt<FMT>;
  const float d = (float)*(const _Float16 *)blk;
  if constexpr (FMT == kFmtQ8_0) return d * (float)(int8_t)blk[F::HDR + e];
  if constexpr (FMT == kFmtQ2_0)
    return d * (float)((blk[F::HDR + (e >> 2)] >> (2 * (e & 3))) & 3) + (float)*(const _Float16 *)(blk + 2);
  const int byte = blk[F::HDR + (e & 15)];
  const int n = e < 16 ? (byte & 15) : (byte >> 4);
  if constexpr (FMT == kFmtQ4_0) return d * (float)(n - 8);
  return d * (float)n + (float)*(const _Float16 *)(blk + 2);
}

// Uniform-weights fallback of common.rs:806-813 for a block cache: out = mean of the attended V rows.
template <int FMT>
struct BlockFallback {
  static constexpr bool kHandlesRow = true;
  static __device__ bool run(const DecodeParams &p, int b, int h, int D) {
    using F = BlockFmt<FMT>;
    const int kvh = h / p.group;
    const uint8_t *vb = (const uint8_t *)p.v + ((int64_t)b * p.kv_bs + (int64_t)kvh * p.head_stride) / 32 * F::BB;
    const int32_t *idx = p.kv_index ? p.kv_index + (int64_t)b * p.index_bs : nullptr;
    const float u = 1.0f / (float)p.len;
    for (int c = threadIdx.x; c < D; c += blockDim.x) {
      float acc = 0.0f;
      for (int t = 0; t < p.len; ++t) {
        const int64_t slot = idx ? (int64_t)min((uint32_t)idx[t], (uint32_t)(p.slot_bound - 1)) : (p.kv_start + t);
        acc += u * block_elem<FMT>(vb + (slot * p.row_stride / 32 + c / 32) * F::BB, c % 32);
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
    return true;
  }
};

constexpr int kWaves = 4;

template <int D>
struct BlockShape {
  static constexpr int KK = D / 32;                       // blocks per row
  static constexpr int VSEG = (D + 127) / 128;            // V pieces per lane per row
  // Channels a lane takes from a V piece: all 8, or at head_dim 64 (where 8 lanes would cover the
  // row and the other 8 repeat them) half a piece: lanes r < 8 the low nibbles / first code dword,
  // lanes r >= 8 the high nibbles / second dword.
  static constexpr int VCH = (D == 64) ? 4 : 8;
  static constexpr int NACC = VCH * VSEG;                 // O accumulators (float4 each)
  static constexpr int MAXH = (D == 256) ? 8 : 16;        // query heads per KV head (bounds the merge LDS)
};

// The wave-private LDS copy of a streamed tile (see the kernel): requests of kLW dwords per lane,
// NLD of them per tile, and the dwords one copy takes.
// Cache policy of the streamed row requests: every byte is read once, so the lines are marked for
// early replacement (q4_0 0.69 -> 0.73, q8_0 0.75 -> 0.82 of HBM peak against the default policy).
constexpr int kStreamPolicy = 2;

template <int FMT, int D, int TW>
struct StreamCopy {
  static constexpr int kLW = 2;
  static constexpr int kRowDwords = (D / 32) * BlockFmt<FMT>::BB / 4;
  static constexpr int NLD = (16 * TW * kRowDwords + 64 * kLW - 1) / (64 * kLW);
  static constexpr int kDwords = NLD * 64 * kLW + 4;  // the last request may run past the tile; a piece's second dword past a row
};

// Waves per SIMD the register allocation aims at: 4 at head_dim 64 (128 registers), 3 at 128 (168;
// q8_0 would spill there and stays at 2, as does the arm with two sets of output accumulators), 2 at 256.  Without the bound most instantiations came out a
// few registers on one or the other side of a step depending on unrelated edits (q4_0 at 128: 165 or
// 170 registers; q8_0 at 256: 256 or 257).
// TOKCOL = 1 (at most four query heads per KV head): the logits MFMA takes the
// query as its row operand, head r / 4 in row r (its high part in the first of a head's four rows,
// its low part in the second, zeros in the others), and the codes as its column operand, so result
// lane (g, n) holds token n of the tile for head g (the two partial dot products in registers 0 and
// 1).  Lane group g keeps head g: the token's block scales are the lane's own (no exchange), the
// softmax runs once per logit instead of once per operand column, a head's maximum is a reduction
// inside one 16-lane row, and the probabilities reach the P operand's layout (lane (j, r): tokens
// 4j..4j+3 of head r % 4) through 256 bytes of LDS per wave.
// TOKCOL = 2 (head_dim 64 and 128, five to eight heads per KV head): the query rows are head r / 2, high part
// in the even row and low part in the odd one, so lane group g keeps the two heads 2g and 2g + 1 (HL
// = 2 logits per lane and tile); the P operand has head r % 4 + 4 (r / 8) in row r, scaled for block
// r / 4 % 2 -- with two blocks per row the sixteen rows are exactly eight heads times two blocks.
// At head_dim 128 (four blocks per row) the output MFMAs run twice, for heads 0..3 and 4..7.
//
// STREAM (rows packed back to back, no index list): a wave's tile is one contiguous run of bytes.
// The per-lane block requests of the other path put a header and 16 or 32 code bytes at an 18- or
// 34-byte stride under every lane, which the texture path serves lane by lane: the q4_0 kernel made
// as many L1 accesses as the F16 kernel for 3.6 times fewer bytes (17 per 128-byte line, counter
// TCP_TOTAL_CACHE_ACCESSES against TCP_TCC_READ_REQ).  Here the lanes fetch consecutive 8-byte pieces
// of the run, park them in a wave-private LDS copy of the tile, and every lane then reads the pieces
// of its MFMA operands straight from there: no trades between lanes at all.
template <int FMT, int D, int TW, bool SOFTCAP, bool INDEXED, int TOKCOL, bool STREAM>
__global__ __launch_bounds__(64 * kWaves, (D == 64) ? 4 : (D == 128) ? ((FMT == kFmtQ8_0 || TOKCOL == 2) ? 2 : 3) : 2) void decode_blocks_kernel(const DecodeParams p) {
  using F = BlockFmt<FMT>;
  using SH = BlockShape<D>;
  using CD = Codec<FMT>;
  constexpr int KK = SH::KK, VSEG = SH::VSEG, NACC = SH::NACC, VCH = SH::VCH;
  constexpr int TILE = 16 * TW;  // tokens per wave iteration
  constexpr float kLn2 = 0.6931471805599453f, kLog2e = 1.4426950408889634f;
  const float inv_cap = SOFTCAP ? 1.0f / p.softcap : 0.0f;

  const int split = blockIdx.x, kvh = blockIdx.y, b = blockIdx.z;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int j = lane >> 4, r = lane & 15;
  const int G = p.group;
  // Head whose query this lane's operand row (or column) carries.  TOKCOL: rows 4g..4g+3 all carry
  // head g, so the four registers of a result lane in lane group g all hold head g's logit and no
  // register has to be picked; the P operand of the output MFMAs has head r % 4 in row r.
  constexpr int HL = (TOKCOL == 2) ? 2 : 1;  // heads a lane keeps logits of
  static_assert(TOKCOL != 2 || D == 64 || D == 128, "two heads per lane: head_dim 64 and 128");
  // P operands of the output MFMAs: one set of sixteen rows, or (two heads per lane at head_dim 128,
  // where a row's four blocks leave room for four heads only) two sets, heads 0..3 and 4..7, over the
  // same V operands and with accumulators of their own.
  constexpr int NQ = (TOKCOL == 2 && D == 128) ? 2 : 1;
  const int rh = (TOKCOL == 2) ? (r >> 1) : (TOKCOL ? (r >> 2) : r);
  const int ph = (TOKCOL == 2) ? (r & 1) : (r & 3);                  // which part of the query the row carries
  const int pa_head = (TOKCOL == 2 && D == 64) ? (r & 3) + 4 * (r >> 3) : (r & 3);  // head in row r of the P operand (set q: + 4 q)
  static_assert(!(STREAM && INDEXED), "an index list gathers rows: they are read block by block");

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

  // K rows are read one whole block per lane and traded between the lane groups (load_block,
  // block_to_pieces).  A wave-wide request covers 16 rows x 4 blocks: one 16-token tile at
  // head_dim 128, half of one at 256 (two requests per tile), both tiles of an iteration at 64
  // (lane group j takes block j % 2 of tile j / 2).
  static_assert(D != 64 || TW == 2 || (TW == 4 && TOKCOL && STREAM), "head_dim 64 pairs the two tiles of an iteration in one request; streamed, tokens as columns: four tiles");
  constexpr int KQ = (D == 64) ? 1 : KK / 4;        // requests per tile (head_dim 64: per iteration)
  constexpr int KL = (D == 64) ? 1 : TW * KQ;
  RawBlock<FMT> kblk[KL];
  // ... and for the 4-bit formats the V rows too: lane (j, r) takes block r/4 (of the request's four)
  // of token 4j + r%4, and the lanes trade dwords through a wave-private strip of LDS (16 bytes per
  // lane, plus 16 bytes after every 16 lanes so that the four lane groups read different banks).
  // head_dim 64: lanes r < 8 take tile 0, the others tile 1.  q8_0 V rows are read in 8-byte pieces.
  constexpr bool kStageV = FMT != kFmtQ8_0;
  constexpr int VL = (D == 64) ? 1 : TW * VSEG;
  RawPiece<FMT> vraw[TW][VSEG][kStageV ? 1 : 4];
  RawBlock<FMT> vblk_raw[kStageV ? VL : 1];
  // STREAM: the tile as dwords in flight, and its LDS copy per wave (K and V apart, so the V copy
  // can be made while the K pieces are still being read).  A request past the attended rows returns
  // zeros (bounds-checked descriptor), so every request is unconditional here too.
  constexpr int RBY = KK * F::BB;                  // bytes per packed row
  static_assert(RBY % 4 == 0, "rows are whole dwords");
  constexpr int RD = RBY / 4;                      // dwords per row
  // A request fetches LW dwords per lane, 256 LW contiguous bytes per wave.  Measured at 1, 2 and 4
  // dwords: 2 was within 1 % of the best for every format (q8_0 +3 % over 1); 4 makes the copies
  // bigger, and with staged scores that leaves room for fewer workgroups (-6 %).
  using SC = StreamCopy<FMT, D, TW>;
  constexpr int LW = SC::kLW, NLD = SC::NLD;
  static_assert(SC::kRowDwords == RD, "launcher and kernel agree on the row");
  uint32_t kst[STREAM ? NLD * LW : 1], vst[STREAM ? NLD * LW : 1];
  // The copies live in the dynamic area behind whatever the token loop keeps there (the staged
  // logits, or the spare slots of lanes that park nothing); the merge at the end reuses all of it.
  constexpr int kTileDw = SC::kDwords;
  extern __shared__ __attribute__((aligned(16))) float dyn_lds[];
  const int stage_row = p.chunk + 4;
  const int staged_heads = p.stage_scores ? p.group : 0;
  // Spare slots of lanes that park no logit: 4 TW floats per lane (tokens as columns: HL TW).
  constexpr int kSparePerLane = TOKCOL ? HL * TW : 4 * TW;
  constexpr int kSpareFloats = 64 * kWaves * kSparePerLane;
  // Tokens as columns: [staged logits][spare slots][tile copies]; tokens as rows: [staged logits, or
  // the spare slots][tile copies] (with staged logits its spare slots are the sink's static stage).
  const int spare_at = (TOKCOL && p.stage_scores) ? staged_heads * stage_row : 0;  // floats
  uint32_t *const tiles = (uint32_t *)(dyn_lds + (TOKCOL ? spare_at + kSpareFloats : (p.stage_scores ? staged_heads * stage_row : kSpareFloats)));
  uint32_t *const k_tile = tiles + wave * kTileDw, *const v_tile = tiles + (kWaves + wave) * kTileDw;
  const uint32_t run_bytes = (uint32_t)min((int64_t)p.len * RBY, (int64_t)0xffffffffll);
  const __amdgpu_buffer_rsrc_t k_rs = __builtin_amdgcn_make_buffer_rsrc((void *)kb, 0, STREAM ? run_bytes : 0u, kBufferFlags);
  const __amdgpu_buffer_rsrc_t v_rs = __builtin_amdgcn_make_buffer_rsrc((void *)vb, 0, STREAM ? run_bytes : 0u, kBufferFlags);
  typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
  // The tile's last request ends with the tile: lanes past it take an offset outside any descriptor
  // (no access, zeros), so no wave fetches bytes of its neighbour's tile.
  constexpr uint32_t kTailAt = (4u * LW) * 64u * (uint32_t)(NLD - 1);
  const uint32_t tail_vo = (kTailAt + (4u * LW) * (uint32_t)lane < (uint32_t)(TILE * RBY)) ? kTailAt + (4u * LW) * (uint32_t)lane : 0x7ffffff0u;
  auto fetch_run = [&](__amdgpu_buffer_rsrc_t rs, int base, uint32_t (&st)[STREAM ? NLD * LW : 1]) {
    const uint32_t off = (uint32_t)min(base, p.len) * (uint32_t)RBY;  // scalar; past the end everything reads as zero
#pragma unroll
    for (int c = 0; c < NLD; ++c) {
      const uint32_t vo = (c == NLD - 1) ? tail_vo : (4u * LW) * (uint32_t)lane + (256u * LW) * (uint32_t)c;
      if constexpr (LW == 4) {
        const u32x4_t v = __builtin_bit_cast(u32x4_t, __builtin_amdgcn_raw_buffer_load_b128(rs, vo, off, kStreamPolicy));
#pragma unroll
        for (int w = 0; w < 4; ++w) st[4 * c + w] = v[w];
      } else if constexpr (LW == 2) {
        const u32x2_t v = __builtin_bit_cast(u32x2_t, __builtin_amdgcn_raw_buffer_load_b64(rs, vo, off, kStreamPolicy));
        st[2 * c] = v[0];
        st[2 * c + 1] = v[1];
      } else {
        st[c] = __builtin_amdgcn_raw_buffer_load_b32(rs, vo, off, kStreamPolicy);
      }
    }
  };
  auto park_run = [&](uint32_t *tile, const uint32_t (&st)[STREAM ? NLD * LW : 1]) {
    wave_lds_fence();  // the reads of the tile before are done
#pragma unroll
    for (int c = 0; c < NLD; ++c) {
      uint32_t *dst = tile + LW * (64 * c + lane);
      if constexpr (LW == 4) *(u32x4_t *)dst = u32x4_t{st[4 * c], st[4 * c + 1], st[4 * c + 2], st[4 * c + 3]};
      else if constexpr (LW == 2) *(u32x2_t *)dst = u32x2_t{st[2 * c], st[2 * c + 1]};
      else *dst = st[c];
    }
    wave_lds_fence();
  };
  // Reads of a parked tile.  The two-dword reads (ds_read2_b32) carry their constant offset in an
  // 8-bit field of dwords, so a lane base reaches 1020 bytes; left to itself the compiler covers the
  // rest of the copy with an address add in front of every read (30 a wave iteration at head_dim 64,
  // where the vector ALU is the limit).  The lane bases are therefore kept as integers the compiler
  // cannot re-derive, one per group of kTilesPerBase tiles, and every read adds a constant that fits.
  constexpr int kRowsAhead = (TOKCOL != 0 && STREAM && D == 64) ? 12 : 3;  // furthest row of a V read past the lane's first (see kSpreadV)
  // (K: a row's blocks lie up to a row further on; V: the base points at the lane's code dword already)
  constexpr auto reads_fit = [](int tiles) {
    return 16 * (tiles - 1) * RBY + RBY <= 1020 && (16 * (tiles - 1) + kRowsAhead) * RBY + 4 * F::CW <= 1020;
  };
  // Where it pays: head_dim 64 (q8_0 apart, which is short of registers and not bound by the vector
  // ALU); elsewhere one base and the compiler's own adds (the pinned bases cost the 128- and
  // 256-wide kernels 8 to 22 registers and some of them spills).
  constexpr bool kPinBases = D == 64 && FMT != kFmtQ8_0;
  constexpr int kTilesPerBase = !kPinBases || reads_fit(TW) ? TW : (TW >= 2 && reads_fit(TW / 2)) ? TW / 2 : 1;
  constexpr int NB = TW / kTilesPerBase;
  static_assert(NB * kTilesPerBase == TW, "groups of tiles divide the iteration");
  // K operand piece of token r of tile tw: code index j of block kk (q2_0: the dword that holds half j)
  uint32_t k_hdr_at = 0, k_code_at[NB] = {};
  if constexpr (STREAM) {
    k_hdr_at = lds_address(k_tile) + 4u * (uint32_t)(r * RD);
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
      k_code_at[nb] = lds_address(k_tile) + 4u * (uint32_t)((16 * kTilesPerBase * nb + r) * RD + ((FMT == kFmtQ2_0) ? (j >> 1) : F::CW * j));
      if constexpr (kPinBases) asm volatile("" : "+v"(k_code_at[nb]));
    }
  }
  auto k_piece = [&](int tw, int kk) {
    RawPiece<FMT> pc;
    const uint32_t blk = (uint32_t)(kk * F::BB);
    const uint32_t row = (uint32_t)(16 * (tw % kTilesPerBase) * RBY);  // bytes from the base's first tile
    const uint32_t code = k_code_at[tw / kTilesPerBase] + row + (blk + (uint32_t)F::HDR) / 4u * 4u;
    if constexpr (F::HDR == 4) {
      pc.hdr = lds_dword(k_hdr_at + (uint32_t)(16 * tw * RBY) + blk);
#pragma unroll
      for (int w = 0; w < F::CW; ++w) pc.code[w] = lds_dword(code + 4u * (uint32_t)w);
    } else {
      pc.hdr = lds_half(k_hdr_at + (uint32_t)(16 * tw * RBY) + blk);
      // with a 2-byte header the code words of every other block straddle dwords
      if ((kk * F::BB) % 4 == 0) {
        uint32_t d[F::CW + 1];
#pragma unroll
        for (int w = 0; w <= F::CW; ++w) d[w] = lds_dword(code + 4u * (uint32_t)w);
#pragma unroll
        for (int w = 0; w < F::CW; ++w) pc.code[w] = __builtin_amdgcn_alignbyte(d[w + 1], d[w], 2u);
      } else {
#pragma unroll
        for (int w = 0; w < F::CW; ++w) pc.code[w] = lds_dword(code + 4u * (uint32_t)w);
      }
    }
    return pc;
  };
  // V piece of token 4j + e of tile tw: block vblk[sg], code index r % 4 (head_dim 64, q8_0: the
  // lane's half of the piece, one dword); the lane's offsets into a row are fixed.
  // Tokens as columns: the contraction slots of the output MFMAs may hold the tile's tokens in any
  // order as long as the P operand follows, and P passes through LDS anyway.  Slot 4j + e is token
  // j + 4e at head_dim 64: one read instruction (fixed e) then takes four neighbouring rows, whose
  // dwords lie side by side in the copy, instead of four rows 4 RD dwords apart (36 dwords for q4_0:
  // lane groups 0 and 1 four banks apart; q4_0 +3..7 % with four heads per KV head and +1..3 % with
  // seven, q4_1 +1..2 %, q2_0 and q8_0 alike).
  // Rows of head_dim 128 span more than half the banks, two lane groups collide wherever their rows
  // lie, and the counters agree: q4_0 the same conflict cycles either way, q8_0 a third more and q2_0
  // 3 % slower with neighbouring rows.
  constexpr bool kSpreadV = TOKCOL != 0 && STREAM && D == 64;
  uint32_t v_blk_byte[VSEG], v_code_dw[VSEG], v_sh[VSEG];
#pragma unroll
  for (int sg = 0; sg < VSEG; ++sg) {
    const uint32_t blk = (uint32_t)(vblk[sg] * F::BB);
    uint32_t a;  // first code byte of the piece
    if constexpr (FMT == kFmtQ2_0) a = blk + 4u + 4u * (uint32_t)((r & 3) >> 1);
    else if constexpr (FMT == kFmtQ8_0 && D == 64) a = blk + (uint32_t)F::HDR + 4u * (uint32_t)(2 * (r & 3) + (r >> 3));
    else a = blk + (uint32_t)F::HDR + 4u * (uint32_t)(F::CW * (r & 3));
    v_blk_byte[sg] = blk;
    v_code_dw[sg] = a / 4;
    v_sh[sg] = a & 3u;
  }
  static_assert(kRowsAhead == (kSpreadV ? 12 : 3), "the furthest row of a V read");
  uint32_t v_hdr_at[VSEG] = {}, v_code_at[NB][VSEG] = {};
  if constexpr (STREAM) {
#pragma unroll
    for (int sg = 0; sg < VSEG; ++sg) {
      const uint32_t first = lds_address(v_tile) + 4u * (uint32_t)((kSpreadV ? j : 4 * j) * RD);  // the lane's first row of tile 0
      v_hdr_at[sg] = first + v_blk_byte[sg];
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) {
        v_code_at[nb][sg] = first + 4u * (uint32_t)(16 * kTilesPerBase * nb * RD) + 4u * v_code_dw[sg];
        if constexpr (kPinBases) asm volatile("" : "+v"(v_code_at[nb][sg]));
      }
    }
  }
  auto v_piece = [&](int tw, int sg, int e) {
    RawPiece<FMT> pc;
    const uint32_t rows = (uint32_t)(kSpreadV ? 4 * e : e);  // rows past the lane's first
    const uint32_t code = v_code_at[tw / kTilesPerBase][sg] + (uint32_t)(16 * (tw % kTilesPerBase) * RBY) + rows * (uint32_t)RBY;
    const uint32_t hdr = v_hdr_at[sg] + (uint32_t)(16 * tw * RBY) + rows * (uint32_t)RBY;
    if constexpr (F::HDR == 4) {
      pc.hdr = lds_dword(hdr);
#pragma unroll
      for (int w = 0; w < F::CW; ++w) pc.code[w] = lds_dword(code + 4u * (uint32_t)w);
    } else if constexpr (FMT == kFmtQ8_0 && D == 64) {  // half a piece: one code dword
      pc.hdr = lds_half(hdr);
      pc.code[0] = __builtin_amdgcn_alignbyte(lds_dword(code + 4u), lds_dword(code), v_sh[sg]);
      pc.code[1] = 0u;
    } else {
      pc.hdr = lds_half(hdr);
      uint32_t d[F::CW + 1];
#pragma unroll
      for (int w = 0; w <= F::CW; ++w) d[w] = lds_dword(code + 4u * (uint32_t)w);
#pragma unroll
      for (int w = 0; w < F::CW; ++w) pc.code[w] = __builtin_amdgcn_alignbyte(d[w + 1], d[w], v_sh[sg]);
    }
    return pc;
  };
  // Rows past the chunk re-read its last row (they are masked below), so every request is
  // unconditional and a tile may be asked for before it is known to exist.
  const int last = t_end - 1;
  // Token -> cache row.  With an index list (INDEXED) the rows of the tile after next are read from
  // the list while the next tile's blocks are requested: the K rows right behind the K requests and
  // the V rows right behind the V requests, so that neither request waits on a load younger than
  // the data it is about to use.
  constexpr int NKR = (D == 64) ? 1 : TW;                               // K rows a lane addresses per iteration
  constexpr int NVR = kStageV ? ((D == 64) ? 1 : TW) : 4 * TW;          // V rows
  const int32_t *idx = INDEXED ? p.kv_index + (int64_t)b * p.index_bs : nullptr;
  // Rows are fetched with plain loads: a slot outside the cache (stale or negative entry of the
  // list) is clamped to the last one, so the list can never steer a load out of the head's slab.
  const uint32_t slot_max = (uint32_t)(p.slot_bound - 1);
  int k_row[INDEXED ? NKR : 1], v_row[INDEXED ? NVR : 1];
  auto k_tok = [&](int base, int i) { return min((D == 64) ? base + 16 * (j >> 1) + r : base + 16 * i + r, last); };
  auto v_tok = [&](int base, int i) {
    if constexpr (!kStageV) return min(base + 16 * (i >> 2) + 4 * j + (i & 3), last);
    else return min((D == 64) ? base + 16 * (r >> 3) + 4 * j + (r & 3) : base + 16 * i + 4 * j + (r & 3), last);
  };
  auto load_idx_k = [&](int base) {
    if constexpr (INDEXED) {
#pragma unroll
      for (int i = 0; i < NKR; ++i) k_row[i] = (int)min((uint32_t)idx[k_tok(base, i)], slot_max);
    }
  };
  auto load_idx_v = [&](int base) {
    if constexpr (INDEXED) {
#pragma unroll
      for (int i = 0; i < NVR; ++i) v_row[i] = (int)min((uint32_t)idx[v_tok(base, i)], slot_max);
    }
  };
  auto k_rowof = [&](int base, int i) -> uint32_t {
    if constexpr (INDEXED) return (uint32_t)k_row[i];
    else return (uint32_t)k_tok(base, i);
  };
  auto v_rowof = [&](int base, int i) -> uint32_t {
    if constexpr (INDEXED) return (uint32_t)v_row[i];
    else return (uint32_t)v_tok(base, i);
  };
  auto load_k = [&](int base) {
    if constexpr (STREAM) {
      fetch_run(k_rs, base, kst);
    } else if constexpr (D == 64) {
      const uint32_t off = __umul24(k_rowof(base, 0), row_bytes);
      kblk[0] = load_block<FMT>(kb, off + (uint32_t)((j & 1) * F::BB));
    } else {
#pragma unroll
      for (int tw = 0; tw < TW; ++tw) {
        const uint32_t off = __umul24(k_rowof(base, tw), row_bytes);
#pragma unroll
        for (int u = 0; u < KQ; ++u) kblk[tw * KQ + u] = load_block<FMT>(kb, off + (uint32_t)((4 * u + j) * F::BB));
      }
    }
  };
  auto load_v = [&](int base) {
    if constexpr (STREAM) {
      fetch_run(v_rs, base, vst);
    } else if constexpr (kStageV && D == 64) {
      const uint32_t off = __umul24(v_rowof(base, 0), row_bytes);
      vblk_raw[0] = load_block<FMT>(vb, off + (uint32_t)(((r >> 2) & 1) * F::BB));
    } else {
#pragma unroll
      for (int tw = 0; tw < TW; ++tw) {
        if constexpr (kStageV) {
          const uint32_t off = __umul24(v_rowof(base, tw), row_bytes);
#pragma unroll
          for (int sg = 0; sg < VSEG; ++sg) vblk_raw[tw * VSEG + sg] = load_block<FMT>(vb, off + (uint32_t)((4 * sg + (r >> 2)) * F::BB));
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const uint32_t off = __umul24(v_rowof(base, 4 * tw + e), row_bytes);
#pragma unroll
            for (int sg = 0; sg < VSEG; ++sg) {
              if constexpr (D == 64) {  // q8_0: the lane's half of the piece is one dword
                const uint32_t blk = off + (uint32_t)(vblk[sg] * F::BB);
                vraw[tw][sg][e].hdr = *(const uint16_t *)(vb + blk);
                vraw[tw][sg][e].code[0] = *(const u32_a2 *)(vb + (blk + (uint32_t)F::HDR + 4u * (uint32_t)(2 * (r & 3) + (r >> 3))));
              } else {
                vraw[tw][sg][e] = load_piece<FMT>(vb, off + (uint32_t)(vblk[sg] * F::BB), (uint32_t)(r & 3));
              }
            }
          }
        }
      }
    }
  };
  const int base0 = t_begin + __builtin_amdgcn_readfirstlane(wave) * TILE;
  load_idx_k(base0);
  load_idx_v(base0);
  load_k(base0);
  load_idx_k(base0 + kWaves * TILE);
  load_v(base0);
  load_idx_v(base0 + kWaves * TILE);
  __builtin_amdgcn_sched_barrier(0);  // keep these requests ahead of the query's

  // ---- Q operand: lane (j, h = r), block kk: the elements slot_elem(j, 0..7), log2 domain, hi + lo.
  // Tokens as columns: row r is head r / 4, and of a head's four rows the first carries the high
  // parts and the second the low parts (the other two are zero), so one MFMA yields both partial
  // dot products, in result registers 0 and 1 of the head's lane group.
  half8_t qh[KK], ql[KK];
  float qsum[KK][HL];   // sum of the scaled query over block kk: the minimum term (tokens as columns: of each head the lane keeps)
  float qinit[KK][HL];  // what a block's MFMA accumulator starts from: -sum over the block of (slot bias + zero point) * q
  {
    const float c = p.scale * 1.4426950408889634f;
    const int h = kvh * G + min(rh, G - 1);
    const float *qp = p.q + (int64_t)b * p.q_bs + (int64_t)h * D;
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
      float qv[8];
#pragma unroll
      for (int s = 0; s < 8; ++s) qv[s] = qp[32 * kk + slot_elem<FMT>(j, s)];  // lanes past the group re-read its last head
      loaded8(qv);
      float part = 0.0f, biased = 0.0f;
#pragma unroll
      for (int s = 0; s < 8; ++s) {
        const float x = (rh < G) ? qv[s] * c : 0.0f;
        part += x;
        if constexpr (FMT == kFmtQ2_0) biased = fmaf(CD::slot_bias(s), x, biased);
        _Float16 hi, lo;
        split_f16(x, hi, lo);
        if constexpr (TOKCOL) {
          qh[kk][s] = (ph == 0) ? hi : ((ph == 1) ? lo : (_Float16)0.0f);
        } else {
          qh[kk][s] = hi;
          ql[kk][s] = lo;
        }
      }
      // the four lane groups hold the four quarters of the block
      part += __shfl_xor(part, 16, 64);
      part += __shfl_xor(part, 32, 64);
      if constexpr (FMT == kFmtQ2_0) {
        biased += __shfl_xor(biased, 16, 64);
        biased += __shfl_xor(biased, 32, 64);
      }
#pragma unroll
      for (int u = 0; u < HL; ++u) {
        // tokens as columns: the sums of the heads whose logits this lane keeps, from a lane whose row is theirs
        const int src = (TOKCOL == 2) ? 4 * j + 2 * u : 4 * j;
        const float head_part = TOKCOL ? __shfl(part, src, 64) : part;
        qsum[kk][u] = head_part;
        if constexpr (FMT == kFmtQ2_0) qinit[kk][u] = -(TOKCOL ? __shfl(biased, src, 64) : biased);
        else qinit[kk][u] = -(CD::kBias + CD::kZero) * head_part;
      }
    }
  }
  // Result lane (j, h) of a logits MFMA holds tokens 4j..4j+3; their block headers were loaded by
  // lanes 16j + (4j + i) (token = lane % 16).
  int hdr_src[4];
  // q2_0: which 16-bit half of a code dword is this lane's K piece (code index j)
  const uint32_t k_sel = q2_half_selector(j & 1);
  // q2_0 V pieces of two tokens side by side (scaled_pair_q2): byte h of the lane's piece (code index
  // r % 4; head_dim 64: the one byte of its half piece) in both code dwords
  uint32_t v_pair_sel[2];
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const uint32_t at = (D == 64) ? (uint32_t)(2 * (r & 1) + (r >> 3)) : (uint32_t)(2 * (r & 1) + h);
    v_pair_sel[h] = 0x0c000c00u | at | ((4u + at) << 16);
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) hdr_src[i] = 4 * (20 * j + i);  // ds_bpermute byte address

  float4_t o_acc[NQ * NACC];  // (set q at q * NACC)
#pragma unroll
  for (int a = 0; a < NQ * NACC; ++a) o_acc[a] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
  // sum over tokens of p * d (q4_0: times -8 it is the zero-point term of the lane's channels) or
  // of p * m (q4_1: the minimum term), per V piece; one more MFMA column each
  constexpr bool kHdrTerm = FMT != kFmtQ8_0;
  // Tokens as columns: the sixteen rows of the P operand are four heads (row % 4) times four copies,
  // and copy row / 4 is multiplied by the scale d of the block that output columns 4 (row / 4) ..
  // + 3 belong to (head_dim 64: two blocks, copies row / 4 % 2).  The V operand is then the bare
  // code, bias + n, with no arithmetic per value; column c of the result is right in the rows of
  // its own block's copy, and the merge reads it from there.  h_acc sums the scaled weights (times
  // -(bias + zero point) it takes the bias back out), m_acc the plain weights times the minimum.
  constexpr bool kScaleP = TOKCOL;
  constexpr bool kMinTerm = kScaleP && F::kHasMin;
  float4_t h_acc[NQ * VSEG], m_acc[kMinTerm ? NQ * VSEG : 1];  // (set q at q * VSEG)
#pragma unroll
  for (int sg = 0; sg < NQ * VSEG; ++sg) h_acc[sg] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
  for (int sg = 0; sg < (kMinTerm ? NQ * VSEG : 1); ++sg) m_acc[sg] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
  float m_run[HL], l_run[HL];  // per (lane = head r; tokens as columns: the HL heads of the lane group); l is this lane group's partial sum
#pragma unroll
  for (int u = 0; u < HL; ++u) m_run[u] = kNegInf, l_run[u] = 0.0f;
  // Dynamic LDS: the chunk's logits when they are staged (p.stage_scores: G rows of chunk + 4 floats),
  // then the merge area.
  using Sink = LogitSink<(TW > 2) ? 2 : TW>;  // (the tokens-as-columns arm only takes its descriptor from it)
  constexpr bool kSinkStage = !TOKCOL;  // (the tokens-as-columns arms store single logits: no static LDS for the sink)
  __shared__ __attribute__((aligned(16))) float logit_stage[kSinkStage ? kWaves : 1][kSinkStage ? Sink::kStageFloats : 4];
  // Lanes that park nothing write to spare slots: in the dynamic area (see `tiles`), or, tokens as
  // rows with staged logits, in the sink's stage (the sink is off then).
  static_assert(!kSinkStage || sizeof(logit_stage) >= kSpareFloats * sizeof(float), "room for every lane's spare slots");
  float *spare = TOKCOL ? dyn_lds + spare_at : (p.stage_scores ? &logit_stage[0][0] : dyn_lds);
  const Sink sink(p, logit_stage[kSinkStage ? wave : 0], b, kvh * G, G, lane, t_end);
  int base_last = -(1 << 30);
  __shared__ uint32_t v_strip[kWaves][VL][(kStageV && !STREAM) ? 64 * 4 + 4 * 4 : 1];  // the staged V rows' code words, wave by wave

  for (int base = base0; base < t_end; base += kWaves * TILE) {
    half4_t pa[NQ][TW];
    if constexpr (TOKCOL) {
      // ---- logits: token base + 16 tw + r, head j (HL = 2: heads 2j and 2j + 1) -----------------
      float sc[TW][HL];
      RawPiece<FMT> both[4];  // head_dim 64: lane group g held block g % 2 of tile g / 2
      if constexpr (STREAM) {
        park_run(k_tile, kst);
        load_k(base + kWaves * TILE);  // the dwords are parked: request the wave's next tile
      } else if constexpr (D == 64) block_to_pieces<FMT>(kblk[0], both);
#pragma unroll
      for (int tw = 0; tw < TW; ++tw) {
#pragma unroll
        for (int u = 0; u < HL; ++u) sc[tw][u] = 0.0f;
        RawPiece<FMT> kpc[KK];
        if constexpr (STREAM) {
#pragma unroll
          for (int kk = 0; kk < KK; ++kk) kpc[kk] = k_piece(tw, kk);
        } else if constexpr (D == 64) {
          kpc[0] = both[2 * tw];
          kpc[1] = both[2 * tw + 1];
        } else {
#pragma unroll
          for (int u = 0; u < KQ; ++u) {
            RawPiece<FMT> four[4];
            block_to_pieces<FMT>(kblk[tw * KQ + u], four);
#pragma unroll
            for (int x = 0; x < 4; ++x) kpc[4 * u + x] = four[x];
          }
        }
#pragma unroll
        for (int kk = 0; kk < KK; ++kk) {
          const half8_t kb_op = code_operand<FMT>(kpc[kk], k_sel);
          // sum of (code - zero) * q = sum of operand * q - sum of (bias + zero) * q: the second term
          // is what the accumulator of the high part starts from
          // (head_dim 64, where the vector ALU is the limit and the two accumulator tuples fit; added
          // behind the MFMA elsewhere)
          constexpr bool kStartFromInit = D == 64 && FMT != kFmtQ8_0;
          float4_t dot = {0.0f, 0.0f, 0.0f, 0.0f};
          if constexpr (kStartFromInit) dot = float4_t{qinit[kk][0], 0.0f, (HL == 2) ? qinit[kk][HL - 1] : 0.0f, 0.0f};
          dot = __builtin_amdgcn_mfma_f32_16x16x32_f16(qh[kk], kb_op, dot, 0, 0, 0);
          // ... times the token's scale for this block, which the lane holds itself
          const half2_t dm = __builtin_bit_cast(half2_t, kpc[kk].hdr);
#pragma unroll
          for (int u = 0; u < HL; ++u) {
            // high and low parts: registers 0 and 1 (two heads per lane: 2u and 2u + 1)
            const float mine = kStartFromInit ? dot[2 * u] + dot[2 * u + 1] : (dot[2 * u] + qinit[kk][u]) + dot[2 * u + 1];
            if constexpr (F::kHasMin) sc[tw][u] = fmaf((float)dm[0], mine, fmaf((float)dm[1], qsum[kk][u], sc[tw][u]));
            else sc[tw][u] = fmaf((float)dm[0], mine, sc[tw][u]);
          }
        }
      }
      if constexpr (D != 64) __builtin_amdgcn_sched_barrier(0);  // (see the other arm)
      if constexpr (!STREAM) load_k(base + kWaves * TILE);
      load_idx_k(base + 2 * kWaves * TILE);
      float mt[HL];
#pragma unroll
      for (int u = 0; u < HL; ++u) {
        mt[u] = kNegInf;
#pragma unroll
        for (int tw = 0; tw < TW; ++tw) {
          if constexpr (SOFTCAP) {
            const float sv = sc[tw][u];
            const float capped = softcap_tanh(sv * kLn2, p.softcap, inv_cap) * kLog2e;
            sc[tw][u] = (sv != sv) ? kNegInf : capped;
          }
          if (base + 16 * tw + r >= t_end) sc[tw][u] = kNegInf;
          sc[tw][u] = fmaxf(sc[tw][u], kNegInf);  // NaN logit counts as -inf (common.rs:790-795)
          mt[u] = fmaxf(mt[u], sc[tw][u]);
        }
      }
      // Emitted logits: parked in the chunk's LDS rows (lanes with nothing to park write to a spare
      // slot of their own), or stored through the sink's bounds-checked descriptor with an offset
      // that drops the store.  Under a uniform branch: calls without scores run 2 % faster that way
      // than with the stores always issued and dropped.
      if (p.scores) {  // uniform
#pragma unroll
        for (int u = 0; u < HL; ++u) {
          const int hj = HL * j + u;  // the head within the group
          const bool parks = hj < staged_heads;
          float *dst = parks ? dyn_lds + hj * stage_row + (base - t_begin) + r : spare + kSparePerLane * (int)threadIdx.x + TW * u;
          const uint32_t row_off = (uint32_t)(((int64_t)hj * p.score_stride + r) * 4);
#pragma unroll
          for (int tw = 0; tw < TW; ++tw) {
            const float logit = sc[tw][u] * kLn2;
            dst[parks ? 16 * tw : tw] = logit;
            const bool writes = sink.on && hj < G && base + 16 * tw + r < t_end;
            __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(uint32_t, logit), sink.rsrc,
                                                  writes ? row_off + 4u * (uint32_t)(base + 16 * tw) : Sink::kDropped, 0u, 2);
          }
        }
      }
      // ---- online softmax: a head's tokens are the 16 lanes of one row ---------------------------
      float alpha[HL];
      constexpr int NPD = (TW + 1) / 2;  // dwords that hold a token column's TW weights (two per dword)
      half2_t pk[HL][NPD];
      bool moved = false;
#pragma unroll
      for (int u = 0; u < HL; ++u) {
        const float m_new = fmaxf(m_run[u], group_allreduce_max<16>(mt[u]));
        const float m_ref = (m_new == kNegInf) ? 0.0f : m_new;
        alpha[u] = __builtin_amdgcn_exp2f(m_run[u] - m_ref);
        moved = moved || alpha[u] != 1.0f;
        m_run[u] = m_new;
#pragma unroll
        for (int d2 = 0; d2 < NPD; ++d2) pk[u][d2] = half2_t{(_Float16)0.0f, (_Float16)0.0f};
        float lsum = 0.0f;
#pragma unroll
        for (int tw = 0; tw < TW; ++tw) {
          const float e = __builtin_amdgcn_exp2f(sc[tw][u] - m_ref);  // the row sum takes the unrounded weight
          lsum += e;
          pk[u][tw >> 1][tw & 1] = (_Float16)e;
        }
        l_run[u] = l_run[u] * alpha[u] + lsum;
      }
      if (__builtin_amdgcn_ballot_w64(moved) != 0) {
        // O accumulator register i belongs to head i, whose factor every lane of row i holds (two heads
        // per lane: to head i + 4 (j / 2), kept as slot i % 2 by lane group 2 (j / 2) + i / 2)
#pragma unroll
        for (int q = 0; q < NQ; ++q) {
          // (two sets: register i of set q is head 4q + i, slot i % 2 of lane group 2q + i / 2)
          float al[4];
#pragma unroll
          for (int i = 0; i < 4; ++i)
            al[i] = (HL == 2) ? __shfl(alpha[i & 1], 16 * (2 * (NQ == 2 ? q : (j >> 1)) + (i >> 1)), 64) : __shfl(alpha[0], 16 * i, 64);
#pragma unroll
          for (int a = 0; a < NACC; ++a)
#pragma unroll
            for (int i = 0; i < 4; ++i) o_acc[q * NACC + a][i] *= al[i];
          if constexpr (kHdrTerm) {
#pragma unroll
            for (int sg = 0; sg < VSEG; ++sg)
#pragma unroll
              for (int i = 0; i < 4; ++i) h_acc[q * VSEG + sg][i] *= al[i];
          }
          if constexpr (kMinTerm) {
#pragma unroll
            for (int sg = 0; sg < VSEG; ++sg)
#pragma unroll
              for (int i = 0; i < 4; ++i) m_acc[q * VSEG + sg][i] *= al[i];
          }
        }
      }
      // (token, head) -> the P operand: lane (j, r) wants tokens 4j..4j+3 of the head of its row
      // (kSpreadV: tokens j, j + 4, j + 8, j + 12, so token r is written to place 4 (r % 4) + r / 4)
      __shared__ __attribute__((aligned(16))) uint32_t p_strip[kWaves][NPD][4 * HL][16];  // 64 words per four heads: writes and reads each touch every bank once
      wave_lds_fence();  // the previous iteration's reads are done
#pragma unroll
      for (int u = 0; u < HL; ++u)
#pragma unroll
        for (int d2 = 0; d2 < NPD; ++d2) p_strip[wave][d2][HL * j + u][kSpreadV ? 4 * (r & 3) + (r >> 2) : r] = __builtin_bit_cast(uint32_t, pk[u][d2]);
      wave_lds_fence();
#pragma unroll
      for (int q = 0; q < NQ; ++q)
#pragma unroll
        for (int d2 = 0; d2 < NPD; ++d2) {
          const u32x4_t w = *(const u32x4_t *)&p_strip[wave][d2][pa_head + 4 * q][4 * j];
#pragma unroll
          for (int h2 = 0; h2 < 2; ++h2) {
            const int tw = 2 * d2 + h2;
            if (tw < TW) {
              const uint32_t sel = h2 ? 0x07060302u : 0x05040100u;
              pa[q][tw] = __builtin_bit_cast(half4_t, u32x2_t{__builtin_amdgcn_perm(w[1], w[0], sel), __builtin_amdgcn_perm(w[3], w[2], sel)});
            }
          }
        }
    } else {
    // ---- logits ---------------------------------------------------------------------------------
    float4_t s[TW];
    RawPiece<FMT> both[4];  // head_dim 64: lane group g held block g % 2 of tile g / 2
    if constexpr (STREAM) {
        park_run(k_tile, kst);
        load_k(base + kWaves * TILE);  // the dwords are parked: request the wave's next tile
      } else if constexpr (D == 64) block_to_pieces<FMT>(kblk[0], both);
#pragma unroll
    for (int tw = 0; tw < TW; ++tw) {
      s[tw] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
      RawPiece<FMT> kpc[KK];
      if constexpr (STREAM) {
#pragma unroll
          for (int kk = 0; kk < KK; ++kk) kpc[kk] = k_piece(tw, kk);
        } else if constexpr (D == 64) {
        kpc[0] = both[2 * tw];
        kpc[1] = both[2 * tw + 1];
      } else {
#pragma unroll
        for (int u = 0; u < KQ; ++u) {
          RawPiece<FMT> four[4];
          block_to_pieces<FMT>(kblk[tw * KQ + u], four);
#pragma unroll
          for (int x = 0; x < 4; ++x) kpc[4 * u + x] = four[x];
        }
      }
#pragma unroll
      for (int kp = 0; kp < KK / 2; ++kp) {
        float4_t dot[2];
#pragma unroll
        for (int u = 0; u < 2; ++u) {
          const int kk = 2 * kp + u;
          const half8_t ka = code_operand<FMT>(kpc[kk], k_sel);
          // sum of (code - zero) * q = sum of operand * q - sum of (bias + zero) * q
          const float c0 = qinit[kk][0];
          dot[u] = float4_t{c0, c0, c0, c0};
          dot[u] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ka, qh[kk], dot[u], 0, 0, 0);
          dot[u] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ka, ql[kk], dot[u], 0, 0, 0);
        }
        if constexpr (F::kHasMin) {
          // the header word already holds (d, m): one exchange per token and block
#pragma unroll
          for (int u = 0; u < 2; ++u)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              const half2_t dm = __builtin_bit_cast(half2_t, __builtin_amdgcn_ds_bpermute(hdr_src[i], (int)kpc[2 * kp + u].hdr));
              s[tw][i] = fmaf((float)dm[0], dot[u][i], fmaf((float)dm[1], qsum[2 * kp + u][0], s[tw][i]));
            }
        } else {
          // scales of two blocks travel together
          const int d_pair = (int)__builtin_amdgcn_perm(kpc[2 * kp + 1].hdr, kpc[2 * kp].hdr, 0x05040100u);
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const half2_t dd = __builtin_bit_cast(half2_t, __builtin_amdgcn_ds_bpermute(hdr_src[i], d_pair));
            s[tw][i] = fmaf((float)dd[0], dot[0][i], fmaf((float)dd[1], dot[1][i], s[tw][i]));
          }
        }
      }
    }
    // Scheduling only: with the requests kept behind the logits the head_dim 128 and 256 kernels run
    // faster (q2_0 at 128: 146 against 173 us, q4_0 at 256: 137 against 146 us, 32K tokens), the
    // head_dim 64 kernels slower (q4_0: 86 against 82 us).
    if constexpr (D != 64) __builtin_amdgcn_sched_barrier(0);
    if constexpr (!STREAM) load_k(base + kWaves * TILE);  // the K registers are free again: request the wave's next tile
    load_idx_k(base + 2 * kWaves * TILE);
    if constexpr (SOFTCAP) {
      // cap * tanh(logit / cap) on the natural-unit logit (flash_attn_f32_f16.cl:563-565), back to log2 units
#pragma unroll
      for (int tw = 0; tw < TW; ++tw)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float sv = s[tw][i];
          const float capped = softcap_tanh(sv * kLn2, p.softcap, inv_cap) * kLog2e;
          s[tw][i] = (sv != sv) ? kNegInf : capped;
        }
    }
    const bool full = base + TILE <= t_end;
    if (!full) {  // uniform: only the chunk's last tile has rows to mask
#pragma unroll
      for (int tw = 0; tw < TW; ++tw)
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (base + 16 * tw + 4 * j + i >= t_end) s[tw][i] = kNegInf;
    }
    float mt = kNegInf;
#pragma unroll
    for (int tw = 0; tw < TW; ++tw)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        s[tw][i] = fmaxf(s[tw][i], kNegInf);  // NaN logit counts as -inf (common.rs:790-795)
        mt = fmaxf(mt, s[tw][i]);
      }
    // Staged or not, the iteration issues the sink's one store (dropped when it has nothing to write):
    // a store on one side of a branch only would make the compiler's wait counts inexact.
    stage_logits<TW>(dyn_lds, stage_row, r, j, staged_heads, base - t_begin, s, spare);
    sink.store(s, base);
    base_last = base;

    // ---- online softmax: the running max of a head is shared by the four lane groups -----------
    mt = rows_allreduce_max(mt);
    const float m_new = fmaxf(m_run[0], mt);
    const float m_ref = (m_new == kNegInf) ? 0.0f : m_new;
    const float alpha = __builtin_amdgcn_exp2f(m_run[0] - m_ref);
    m_run[0] = m_new;
    float lsum = 0.0f;
#pragma unroll
    for (int tw = 0; tw < TW; ++tw) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        // The row sum takes the unrounded weight: it also normalises the emitted scores, and over
        // a handful of tokens the f16 roundings of the weights (2^-12 each) would not average out.
        const float e = __builtin_amdgcn_exp2f(s[tw][i] - m_ref);
        lsum += e;
        pa[0][tw][i] = (_Float16)e;
      }
    }
    l_run[0] = l_run[0] * alpha + lsum;
    if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0) {
      // O accumulator register i of lane group j belongs to head 4j + i: fetch that head's factor.
      float al[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) al[i] = __shfl(alpha, 4 * j + i, 64);
#pragma unroll
      for (int a = 0; a < NACC; ++a)
#pragma unroll
        for (int i = 0; i < 4; ++i) o_acc[a][i] *= al[i];
      if constexpr (kHdrTerm) {
#pragma unroll
        for (int sg = 0; sg < VSEG; ++sg)
#pragma unroll
          for (int i = 0; i < 4; ++i) h_acc[sg][i] *= al[i];
      }
    }

    }

    // ---- O += P . V -----------------------------------------------------------------------------
    if constexpr (STREAM) {
      park_run(v_tile, vst);
      load_v(base + kWaves * TILE);
    }
    // The operands of tile tw, V piece sg: bv[c] = channel slot c of the lane's four tokens, hv = their
    // d (or m) for the header term; with the scales on the P side: bv[c] = the bare codes, dv = the
    // tokens' d, hv = their m.
    auto v_operands = [&](int tw, int sg, half4_t (&bv)[VCH], half4_t &hv, half4_t &dv) {
        RawPiece<FMT> vpc[4];  // the lane's piece of tokens 4j .. 4j+3
        if constexpr (STREAM) {
#pragma unroll
          for (int e = 0; e < 4; ++e) vpc[e] = v_piece(tw, sg, e);
        } else if constexpr (kStageV) {
          constexpr bool kShared = D == 64;  // one request serves both tiles
          const RawBlock<FMT> &mine = vblk_raw[kShared ? 0 : tw * VSEG + sg];
          uint32_t *strip = v_strip[wave][kShared ? 0 : tw * VSEG + sg];
          // The lanes of a wave exchange data through the strip, so the write must be ordered before
          // the other lanes' reads and those before the next write: wave-level fences (LDS operations
          // of a wave execute in order; the fences are there for the compiler, which may otherwise
          // move a lane's reads above its own write, since it reads addresses it did not write).
          if (!kShared || tw == 0) {
            wave_lds_fence();  // the previous reads of this strip are done
            if constexpr (FMT == kFmtQ2_0) *(u32x4_t *)(strip + 4 * lane + 4 * j) = u32x4_t{mine.code[0], mine.code[1], 0u, 0u};
            else *(u32x4_t *)(strip + 4 * lane + 4 * j) = u32x4_t{mine.code[0], mine.code[1], mine.code[2], mine.code[3]};
            wave_lds_fence();
          }
          // token 4j + e was loaded by lane 16j + 4(r/4) + e (head_dim 64: 16j + 8 tw + 4(r/4 % 2) + e);
          // this lane wants dword r%4 of it
          const int quad = kShared ? 2 * tw + ((r >> 2) & 1) : (r >> 2);
          const uint32_t *src = strip + 68 * j + 16 * quad + ((FMT == kFmtQ2_0) ? ((r & 3) >> 1) : (r & 3));  // q2_0: the dword with half r%4
#pragma unroll
          for (int e = 0; e < 4; ++e) vpc[e].code[0] = src[4 * e];
          // header of token 4j + e: lane e of that quad has it (head_dim 64: the quad may sit 8 lanes away)
          int own_hdr = (int)mine.hdr;
          if constexpr (kShared) {
            const int other = __builtin_amdgcn_update_dpp(0, own_hdr, 0x128, 0xf, 0xf, false);  // row_ror:8
            own_hdr = ((r >> 3) == tw) ? own_hdr : other;
          }
          vpc[0].hdr = (uint32_t)__builtin_amdgcn_update_dpp(0, own_hdr, 0x00, 0xf, 0xf, false);
          vpc[1].hdr = (uint32_t)__builtin_amdgcn_update_dpp(0, own_hdr, 0x55, 0xf, 0xf, false);
          vpc[2].hdr = (uint32_t)__builtin_amdgcn_update_dpp(0, own_hdr, 0xaa, 0xf, 0xf, false);
          vpc[3].hdr = (uint32_t)__builtin_amdgcn_update_dpp(0, own_hdr, 0xff, 0xf, 0xf, false);
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e) vpc[e] = vraw[tw][sg][e];
        }
        // The V operand of channel c wants the four tokens' values side by side: the code words of two
        // tokens are interleaved before the codes come out (scaled_pair*), so a register holds one
        // channel of two tokens and no value is moved afterwards.
        half2_t vpair[2][VCH];
        if constexpr (FMT == kFmtQ2_0) {
          scaled_pair_q2<VCH, !kScaleP>(vpc[0], vpc[1], v_pair_sel, vpair[0]);
          scaled_pair_q2<VCH, !kScaleP>(vpc[2], vpc[3], v_pair_sel, vpair[1]);
        } else if constexpr (FMT == kFmtQ8_0) {
          scaled_pair_q8<VCH, !kScaleP>(vpc[0], vpc[1], vpair[0]);
          scaled_pair_q8<VCH, !kScaleP>(vpc[2], vpc[3], vpair[1]);
        } else {
          scaled_pair<FMT, VCH, !kScaleP>(vpc[0], vpc[1], (uint32_t)(r >> 3), vpair[0]);
          scaled_pair<FMT, VCH, !kScaleP>(vpc[2], vpc[3], (uint32_t)(r >> 3), vpair[1]);
        }
        if constexpr (kHdrTerm && (!kScaleP || F::kHasMin)) {
          // d (q4_0: low halves of the headers) or m (q4_1, q2_0: high halves) of the lane's four tokens
          constexpr uint32_t sel = F::kHasMin ? 0x07060302u : 0x05040100u;
          const uint32_t h01 = __builtin_amdgcn_perm(vpc[1].hdr, vpc[0].hdr, sel);
          const uint32_t h23 = __builtin_amdgcn_perm(vpc[3].hdr, vpc[2].hdr, sel);
          hv = __builtin_bit_cast(half4_t, u32x2_t{h01, h23});
        }
        if constexpr (kScaleP) {
          const uint32_t d01 = __builtin_amdgcn_perm(vpc[1].hdr, vpc[0].hdr, 0x05040100u);
          const uint32_t d23 = __builtin_amdgcn_perm(vpc[3].hdr, vpc[2].hdr, 0x05040100u);
          dv = __builtin_bit_cast(half4_t, u32x2_t{d01, d23});
        }
#pragma unroll
        for (int c = 0; c < VCH; ++c) bv[c] = half4_t{vpair[0][c][0], vpair[0][c][1], vpair[1][c][0], vpair[1][c][1]};
    };
    const half4_t ones = {(_Float16)1.0f, (_Float16)1.0f, (_Float16)1.0f, (_Float16)1.0f};
    if constexpr (TW == 2 && TOKCOL && D == 128) {
      // Both tiles in one MFMA of 32 tokens (it holds the matrix core no longer than one of 16):
      // contraction slots 0..3 of a lane are its four tokens of the first tile, 4..7 of the second.
      // (The tokens-as-rows arm has no registers for the operands of two tiles at once; head_dim 64
      // ran 2 % slower this way.)
      auto both = [](half4_t a, half4_t b) { return half8_t{a[0], a[1], a[2], a[3], b[0], b[1], b[2], b[3]}; };
#pragma unroll
      for (int sg = 0; sg < VSEG; ++sg) {
        half4_t bv0[VCH], bv1[VCH], hv0 = {}, hv1 = {}, dv0 = {}, dv1 = {};
        v_operands(0, sg, bv0, hv0, dv0);
        v_operands(1, sg, bv1, hv1, dv1);
#pragma unroll
        for (int q = 0; q < NQ; ++q) {
          const half8_t pw = both(pa[q][0], pa[q][1]);
          half8_t pv = pw;
          if constexpr (kScaleP) {
            pv = both(pa[q][0] * dv0, pa[q][1] * dv1);
            if constexpr (kHdrTerm) h_acc[q * VSEG + sg] = __builtin_amdgcn_mfma_f32_16x16x32_f16(pv, both(ones, ones), h_acc[q * VSEG + sg], 0, 0, 0);
            if constexpr (kMinTerm) m_acc[q * VSEG + sg] = __builtin_amdgcn_mfma_f32_16x16x32_f16(pw, both(hv0, hv1), m_acc[q * VSEG + sg], 0, 0, 0);
          } else if constexpr (kHdrTerm) {
            h_acc[sg] = __builtin_amdgcn_mfma_f32_16x16x32_f16(pw, both(hv0, hv1), h_acc[sg], 0, 0, 0);
          }
#pragma unroll
          for (int c = 0; c < VCH; ++c)
            o_acc[q * NACC + sg * VCH + c] = __builtin_amdgcn_mfma_f32_16x16x32_f16(pv, both(bv0[c], bv1[c]), o_acc[q * NACC + sg * VCH + c], 0, 0, 0);
        }
      }
    } else {
#pragma unroll
      for (int tw = 0; tw < TW; ++tw)
#pragma unroll
        for (int sg = 0; sg < VSEG; ++sg) {
          half4_t bv[VCH], hv = {}, dv = {};
          v_operands(tw, sg, bv, hv, dv);
          static_assert(NQ == 1 || (TW == 2 && D == 128), "two sets of P operands come with the 32-token MFMAs");
          half4_t pv = pa[0][tw];
          if constexpr (kScaleP) {
            pv = pa[0][tw] * dv;
            if constexpr (kHdrTerm) h_acc[sg] = __builtin_amdgcn_mfma_f32_16x16x16f16(pv, ones, h_acc[sg], 0, 0, 0);
            if constexpr (kMinTerm) m_acc[sg] = __builtin_amdgcn_mfma_f32_16x16x16f16(pa[0][tw], hv, m_acc[sg], 0, 0, 0);
          } else if constexpr (kHdrTerm) {
            h_acc[sg] = __builtin_amdgcn_mfma_f32_16x16x16f16(pa[0][tw], hv, h_acc[sg], 0, 0, 0);
          }
#pragma unroll
          for (int c = 0; c < VCH; ++c) o_acc[sg * VCH + c] = __builtin_amdgcn_mfma_f32_16x16x16f16(pv, bv[c], o_acc[sg * VCH + c], 0, 0, 0);
        }
    }
    if constexpr (!STREAM) load_v(base + kWaves * TILE);
    load_idx_v(base + 2 * kWaves * TILE);
  }
  if (p.stage_scores) {
    flush_staged_logits(p, dyn_lds, stage_row, b, kvh * G, G, t_begin, t_end);
  } else {
    if constexpr (!TOKCOL) sink.store_tail(base_last);  // (TOKCOL stores single logits: no group is cut)
    __syncthreads();  // the other waves' spare slots lie in the merge area
  }

  if constexpr (kScaleP && kHdrTerm) {
#pragma unroll
    for (int q = 0; q < NQ; ++q)
#pragma unroll
      for (int sg = 0; sg < VSEG; ++sg)
#pragma unroll
        for (int c = 0; c < VCH; ++c) {
          const float bias = (D == 64) ? half_slot_bias<FMT>(c) : CD::slot_bias(c);
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            float o = fmaf(-(bias + CD::kZero), h_acc[q * VSEG + sg][i], o_acc[q * NACC + sg * VCH + c][i]);
            if constexpr (kMinTerm) o += m_acc[q * VSEG + sg][i];
            o_acc[q * NACC + sg * VCH + c][i] = o;
          }
        }
  } else if constexpr (kHdrTerm) {
    constexpr float kTerm = (FMT == kFmtQ4_0) ? -CD::kZero : 1.0f;
#pragma unroll
    for (int sg = 0; sg < VSEG; ++sg)
#pragma unroll
      for (int c = 0; c < VCH; ++c)
#pragma unroll
        for (int i = 0; i < 4; ++i) o_acc[sg * VCH + c][i] = fmaf(kTerm, h_acc[sg][i], o_acc[sg * VCH + c][i]);
  }

  // ---- merge: lane groups (row sum), then the waves through LDS ---------------------------------
  if constexpr (TOKCOL) {
#pragma unroll
    for (int u = 0; u < HL; ++u) l_run[u] = group_allreduce_sum<16>(l_run[u]);  // lane group j holds head j (heads 2j, 2j + 1)
  } else {
    l_run[0] += __shfl_xor(l_run[0], 16, 64);
    l_run[0] += __shfl_xor(l_run[0], 32, 64);
  }
  const int own_copy = (D == 64) ? ((r >> 2) & 1) : (r >> 2);  // the P copy scaled for this lane's output columns
  float (*lds_m)[16] = (float (*)[16])dyn_lds;
  float (*lds_l)[16] = lds_m + kWaves;
  constexpr int MH = TOKCOL ? 4 * HL : SH::MAXH;  // heads a workgroup merges (tokens as columns: groups of up to four or eight)
  float (*lds_acc)[MH][D + 4] = (float (*)[MH][D + 4])(dyn_lds + 2 * kWaves * 16);
  if (TOKCOL ? r == 0 : j == 0) {
#pragma unroll
    for (int u = 0; u < HL; ++u) {
      lds_m[wave][TOKCOL ? HL * j + u : r] = m_run[u];
      lds_l[wave][TOKCOL ? HL * j + u : r] = l_run[u];
    }
  }
#pragma unroll
  for (int sg = 0; sg < VSEG; ++sg)
#pragma unroll
    for (int c = 0; c < VCH; ++c) {
      const int ch = 32 * vblk[sg] + ((D == 64) ? half_slot_elem<FMT>(r & 3, r >> 3, c) : slot_elem<FMT>(r & 3, c));
#pragma unroll
      for (int i = 0; i < 4; ++i)
        // (tokens as columns: row 4j + i is head i scaled for block j; two heads per lane at head_dim 64:
        // head i + 4 (j / 2) scaled for block j % 2, at 128: set q holds head 4q + i)
#pragma unroll
        for (int q = 0; q < NQ; ++q)
          if ((TOKCOL == 2 && D == 64) ? (j & 1) == own_copy : (TOKCOL ? j == own_copy : 4 * j + i < MH))
            lds_acc[wave][(TOKCOL == 2 && D == 64) ? i + 4 * (j >> 1) : (TOKCOL ? 4 * q + i : 4 * j + i)][ch] = o_acc[q * NACC + sg * VCH + c][i];
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
  constexpr int TW = (D == 256) ? 1 : 2;  // head_dim 256 at two tiles needs every register (one wave per SIMD)
  // Head_dim 64, rows streamed, tokens as columns: four tiles (64 tokens) per wave iteration -- its
  // rows are half as long, and the softmax and the exchanges of an iteration cost the same.
  constexpr int TW64 = 4;
  const bool cap = p.softcap > 0.0f, indexed = p.kv_index != nullptr;
  // Two heads per lane (see the kernel).  At head_dim 128 only without scores: with them the arm's
  // single-float logit stores (two per lane and tile) make it 8-16 % slower than the tokens-as-rows arm.
  const bool wide = (D == 64 || (D == 128 && p.scores == nullptr)) && p.group > 4 && p.group <= 8;
  const bool tokcol = p.group <= 4 || wide;
  // Packed rows without an index list are streamed (see the kernel); the slabs must start on a dword.
  const int64_t head_blocks = ((int64_t)p.kv_bs | (int64_t)p.head_stride) / 32;
  // (Measured per arm: q8_0 +10 % either way, q2_0 +10 % and q4_0 +3 % with tokens as columns; the
  // tokens-as-rows arm of the 4-bit formats has no registers left for it at head_dim 128 and 256 and
  // ran 3-5 % slower, at 64 it has and runs 3 % faster.)
  // (A head's run stays under 2 GiB: the offsets past the tile that the kernel hands idle lanes must
  // not wrap when the tile's offset is added.)
  const bool stream_rows = !indexed && p.row_stride == D && (((uintptr_t)p.k | (uintptr_t)p.v) & 3) == 0 &&
                           (int64_t)p.len * (D / 32) * BlockFmt<FMT>::BB < (1ll << 31) &&
                           (head_blocks * BlockFmt<FMT>::BB) % 4 == 0 && (FMT == kFmtQ8_0 || tokcol || D == 64);
  // With scores the chunks are kept short enough for a workgroup's logits to wait in LDS until its
  // token loop is over (kStageBytes; two workgroups per CU still fit beside the V strips or the
  // streamed tiles' LDS copies).
  const bool four_tiles = D == 64 && tokcol && stream_rows;
  const int tile_rows = kWaves * 16 * (four_tiles ? TW64 : TW);
  const int kTileCopies = 2 * kWaves * (four_tiles ? StreamCopy<FMT, D, TW64>::kDwords : StreamCopy<FMT, D, TW>::kDwords) * 4;
  const int kStageBytes = (kTileCopies > 24 * 1024) ? 32 * 1024 : 48 * 1024;
  const size_t merge_bytes = (2 * kWaves * 16 + kWaves * (tokcol ? (wide ? 8 : 4) : BlockShape<D>::MAXH) * (D + 4)) * sizeof(float);
  const int max_chunk = staged_chunk_limit(ctx, p, kStageBytes, tile_rows);
  auto pick = [&](auto tc, auto st) {
    constexpr int TC = decltype(tc)::value;
    constexpr bool ST = decltype(st)::value;
    if constexpr (ST && D == 64 && TC != 0) return cap ? decode_blocks_kernel<FMT, D, TW64, true, false, TC, true> : decode_blocks_kernel<FMT, D, TW64, false, false, TC, true>;
    else if constexpr (ST && (FMT == kFmtQ8_0 || TC != 0 || D == 64)) return cap ? decode_blocks_kernel<FMT, D, TW, true, false, TC, true> : decode_blocks_kernel<FMT, D, TW, false, false, TC, true>;
    else return cap ? (indexed ? decode_blocks_kernel<FMT, D, TW, true, true, TC, false> : decode_blocks_kernel<FMT, D, TW, true, false, TC, false>)
                    : (indexed ? decode_blocks_kernel<FMT, D, TW, false, true, TC, false> : decode_blocks_kernel<FMT, D, TW, false, false, TC, false>);
  };
  typedef std::integral_constant<int, 0> Rows;
  typedef std::integral_constant<int, 1> Cols;
  typedef std::integral_constant<int, (D == 64 || D == 128) ? 2 : 1> Cols2;  // (head_dim 256 has no such arm; `wide` is false there)
  auto kern = stream_rows ? (wide ? pick(Cols2{}, std::true_type{}) : tokcol ? pick(Cols{}, std::true_type{}) : pick(Rows{}, std::true_type{}))
                          : (wide ? pick(Cols2{}, std::false_type{}) : tokcol ? pick(Cols{}, std::false_type{}) : pick(Rows{}, std::false_type{}));
  // dynamic LDS: staged logits or spare slots, then (streamed rows) the tile copies; the merge reuses it
  // (the spare slots of lanes that park no logit: 4 TW floats per lane, tokens as columns HL TW)
  const size_t spare_bytes = 64 * kWaves * sizeof(float) * (tokcol ? (wide ? 2 : 1) * (four_tiles ? TW64 : TW) : 4 * TW);
  const size_t tile_bytes = stream_rows ? (size_t)kTileCopies : 0;
  const size_t staged_spare = tokcol ? spare_bytes : 0;  // tokens as columns keep their spare slots behind the staged logits
  const int wgs_per_cu = argus_wgs_per_cu(ctx, kern, 64 * kWaves,
                                          max_chunk > 0 ? (size_t)kStageBytes + staged_spare + tile_bytes : std::max(merge_bytes, spare_bytes + tile_bytes));
  choose_splits(p, batch * p.n_heads_kv, tile_rows, (int64_t)ctx->compute_units * wgs_per_cu, max_chunk);
  p.direct = 0;
  p.stage_scores = p.scores && p.chunk <= max_chunk;
  const size_t lds_bytes = std::max(merge_bytes, (p.stage_scores ? (size_t)p.group * (p.chunk + 4) * sizeof(float) + staged_spare : spare_bytes) + tile_bytes);
  ARGUS_HIP_CHECK(ctx, argus_raise_lds_limit(ctx, kern, kStageBytes + kTileCopies + (int)spare_bytes + 1024));
  const int rc = reserve_partials(ctx, p, batch, D);
  if (rc != ARGUS_HIP_OK) return rc;
  ctx->plan = argus_hip_decode_plan{p.nsplit, p.chunk, wgs_per_cu, (int32_t)lds_bytes, 2, 2, p.stage_scores};
  KernelTimer timer(ctx, stream);
  hipLaunchKernelGGL(kern, dim3(p.nsplit, p.n_heads_kv, batch), dim3(64 * kWaves), lds_bytes, stream, p);
  timer.mark();
  ARGUS_HIP_CHECK(ctx, hipGetLastError());
  hipLaunchKernelGGL((decode_combine_kernel<BlockFallback<FMT>, D>), combine_grid(p, batch), dim3(256), 0, stream, p);
  ARGUS_HIP_CHECK(ctx, hipGetLastError());
  return ARGUS_HIP_OK;
}

template <int FMT>
int launch_blocks_dim(argus_hip_ctx *ctx, DecodeParams &p, int D, int batch, hipStream_t stream) {
  switch (D) {
    case 64: return launch_blocks<FMT, 64>(ctx, p, batch, stream);
    case 128: return launch_blocks<FMT, 128>(ctx, p, batch, stream);
    case 256: return launch_blocks<FMT, 256>(ctx, p, batch, stream);
    default: return argus_fail(ctx, ARGUS_HIP_ERR_UNSUPPORTED, "attention_gen: head_dim %d not in {64,128,256}", D);
  }
}

}  // namespace

int launch_decode_blocks(argus_hip_ctx *ctx, DecodeParams &p, int D, int kv_dtype, int batch, hipStream_t stream) {
  // The kernels lay rows, partials and LDS out for these three widths; any other would run the
  // wrong instantiation over the caller's buffers.
  if (D != 64 && D != 128 && D != 256)
    return argus_fail(ctx, ARGUS_HIP_ERR_UNSUPPORTED, "attention_gen: head_dim %d not in {64,128,256}", D);
  if (p.group > ((D == 256) ? 8 : 16))
    return argus_fail(ctx, ARGUS_HIP_ERR_UNSUPPORTED, "attention_gen: %d query heads per KV head on a block-quantised cache", p.group);
  if ((p.row_stride % 32) || (p.head_stride % 32) || (p.kv_bs % 32))
    return argus_fail(ctx, ARGUS_HIP_ERR_INVALID, "attention_gen: block-quantised cache strides must be whole 32-element blocks");
  // rows are addressed as (row index, 24 bits) x (row bytes, 24 bits) -> 32-bit byte offset
  const int64_t rows = p.kv_index ? p.slot_bound : p.len;  // an index list may name any slot of the cache
  if (rows >= (1 << 24) || p.row_stride / 32 * 34 >= (1 << 24) || rows * (p.row_stride / 32 * 34) > 0xffffffffll)
    return argus_fail(ctx, ARGUS_HIP_ERR_UNSUPPORTED, "attention_gen: block-quantised head slab beyond 4 GiB");
  if (!score_rows_addressable(p))
    return argus_fail(ctx, ARGUS_HIP_ERR_UNSUPPORTED, "attention_gen: score rows of a head group beyond 2 GiB");
  switch (kv_dtype) {
    case ARGUS_HIP_Q4_0: return launch_blocks_dim<kFmtQ4_0>(ctx, p, D, batch, stream);
    case ARGUS_HIP_Q4_1: return launch_blocks_dim<kFmtQ4_1>(ctx, p, D, batch, stream);
    case ARGUS_HIP_Q2_0: return launch_blocks_dim<kFmtQ2_0>(ctx, p, D, batch, stream);
    case ARGUS_HIP_Q8_0: return launch_blocks_dim<kFmtQ8_0>(ctx, p, D, batch, stream);
    default: return argus_fail(ctx, ARGUS_HIP_ERR_UNSUPPORTED, "attention_gen: kv dtype %d is not a block format", kv_dtype);
  }
}

}  // namespace argus_decode
