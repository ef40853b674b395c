// KIVI fused dequant + decode attention on the matrix cores (Q2 / Q4 / Q8, head_dim 64 / 128).
//
// Same arithmetic as kivi_attn.hip (dequant `code*d + m`, crates/techniques/kivi/src/kivi_attn.cu:
// 213-218, block layouts kivi_attn.cu:256-262 / 357-361), reorganised so the per-element work is
// an unpack, not `Hq/Hkv` FMAs:
//
//   logits  S[t][h] = sum_ch code[ch][t] * (q[h][ch] * d[ch])  +  sum_ch m[ch] * q[h][ch]
//   output  O[h][c] = sum_t (p[h][t] * d[t][cb]) * code[t][c]   +  sum_t p[h][t] * m[t][cb]
//
// Every term is a 16x16x32 f16 MFMA.  The codes are the operand that has 8 contraction values per
// lane (8 channels of one token for the logits, 8 tokens of one channel for the output); KIVI
// stores K per channel and V per token, i.e. both transposed relative to that, so each wave copies
// its unit's K and V tiles (32 tokens) into a private LDS region and gathers the codes with byte
// reads.  A code is turned into an exact f16 integer with one mask-or (1024 + code << shift) and one
// packed subtract; the sub-byte shift is undone as a power-of-two factor on the MFMA result.  The
// block scales go to the *other* operand in f32 (q*d split into f16 hi + lo, p*d in f16), and the
// zero-point terms are MFMAs whose operand is the f16 `m` header itself.  Waves are autonomous:
// no workgroup barrier inside the unit loop.  Residual rows (F32 or F16) run through the same
// MFMAs with the row split into f16 hi + lo.
#include "kivi_common.hpp"

#include <algorithm>

namespace argus_kivi {

using namespace argus_decode;

namespace {

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

__device__ __forceinline__ void wave_lds_fence() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// Two bytes -> two exact f16 integers (code << shift), via 1024 + x in the f16 mantissa.
__device__ __forceinline__ half2_t codes_to_half2(uint32_t b0, uint32_t b1, uint32_t mask2) {
  const uint32_t v = ((b0 | (b1 << 16)) & mask2) | 0x64006400u;
  const half2_t h = __builtin_bit_cast(half2_t, v);
  const half2_t k = {(_Float16)1024.0f, (_Float16)1024.0f};
  return h - k;
}

__device__ __forceinline__ half8_t make_half8(half2_t a, half2_t b, half2_t c, half2_t d) {
  return half8_t{a[0], a[1], b[0], b[1], c[0], c[1], d[0], d[1]};
}

template <int BITS, int D>
__global__ __launch_bounds__(256) void kivi_mfma_kernel(const KiviParams kp) {
  constexpr int BB = 4 + 32 * BITS / 8;  // block bytes
  constexpr int KK = D / 32;             // 32-channel steps == V blocks per token
  constexpr int TILE_BYTES = D * BB;     // one K tile == one V tile
  constexpr int WAVE_BYTES = 2 * TILE_BYTES;
  constexpr int MERGE_BYTES = 4 * 16 * (D + 4) * 4 + 4 * 16 * KK * 4 + 2 * 4 * 16 * 4;
  constexpr int SMEM = (4 * WAVE_BYTES > MERGE_BYTES) ? 4 * WAVE_BYTES : MERGE_BYTES;
  constexpr uint32_t CMASK = (1u << BITS) - 1u;
  constexpr float kLn2 = 0.6931471805599453f;
  constexpr float kOpScale = 64.0f;  // power of two applied to the f16 operands that carry scales
  __shared__ __attribute__((aligned(16))) uint8_t smem[SMEM];

  const DecodeParams &p = kp.d;
  const int split = blockIdx.x, kvh = blockIdx.y, b = blockIdx.z;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int j = lane >> 4, r = lane & 15;
  const int G = p.group;
  const int gpf = kp.res_cap / kUnit;
  const int q_units = kp.q_tokens / kUnit;

  uint8_t *sK = smem + wave * WAVE_BYTES;
  uint8_t *sV = sK + TILE_BYTES;
  const uint8_t *qk_b = kp.qk + (int64_t)b * kp.qk_bs;
  const uint8_t *qv_b = kp.qv + (int64_t)b * kp.qv_bs;

  // ---- constant Q operands: lane (h = r, j) holds channels 32kk + 8j + e -------------------------
  // log2 domain, times kOpScale: the low halves of the f16 hi + lo splits (q, and q*d with d as
  // small as range/255) would otherwise sit in the f16 subnormal range and lose their bits.
  float qf[KK][8];
  half8_t qh[KK], ql[KK];
  {
    const float c = p.scale * 1.4426950408889634f * kOpScale;
    const float *qp = p.q + (int64_t)b * p.q_bs + (int64_t)(kvh * G + min(r, G - 1)) * D;
#pragma unroll
    for (int kk = 0; kk < KK; ++kk)
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float x = (r < G) ? qp[32 * kk + 8 * j + e] * c : 0.0f;
        qf[kk][e] = x;
        _Float16 hi, lo;
        split_f16(x, hi, lo);
        qh[kk][e] = hi;
        ql[kk][e] = lo;
      }
  }

  // Sub-byte position of this lane's token (logit side, token = 16*half + r) and channel (output
  // side, channel = 16*sub + r): both depend on r only.
  const int sh_r = (r * BITS) % 8;
  const uint32_t mask_r = (CMASK << sh_r) * 0x00010001u;
  // undoes the shift on this lane's output columns and the operand scale on p*d
  const float fv = 1.0f / ((float)(1 << sh_r) * kOpScale);

  float4_t o_acc[2 * KK];  // [cb*2 + sub]: lane (j, n=r) reg i -> head 4j+i, channel 32cb+16sub+r
  float4_t m_acc = {0.0f, 0.0f, 0.0f, 0.0f};  // zero-point term: lane (j, n=cb) reg i -> head 4j+i
#pragma unroll
  for (int a = 0; a < 2 * KK; ++a) o_acc[a] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
  float m_run = kNegInf, l_run = 0.0f;
  bool shift_pending = true;  // o_acc still carries the per-lane 2^shift factor

  // token owned by k-slot e of lane group jj (the lane's own logits, in MFMA output order)
  auto tok_of = [](int jj, int e) { return (e < 4) ? (4 * jj + e) : (16 + 4 * jj + (e - 4)); };

  const int u_begin = split * kp.units_per_split;
  const int u_end = min(kp.units_total, u_begin + kp.units_per_split);
  for (int u = u_begin + wave; u < u_end; u += 4) {
    const bool quant = u < q_units;
    float4_t s[2];
    s[0] = s[1] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
    int tok0, n_valid;

    if (quant) {
      tok0 = u * kUnit;
      n_valid = kUnit;
      // ---- stage the unit's K and V tiles into this wave's LDS region ---------------------------
      {
        const int flush = u / gpf, gif = u % gpf;
        const int64_t kblk = ((int64_t)flush * p.n_heads_kv * gpf + (int64_t)kvh * gpf + gif) * D;
        const int tif0 = (u * kUnit) % kp.res_cap;
        const int64_t vblk = (((int64_t)flush * p.n_heads_kv + kvh) * kp.res_cap + tif0) * KK;
        const u32x4_t *ksrc = (const u32x4_t *)(qk_b + kblk * BB);
        const u32x4_t *vsrc = (const u32x4_t *)(qv_b + vblk * BB);
        wave_lds_fence();  // the previous unit's reads are done
#pragma unroll
        for (int c = 0; c < (TILE_BYTES / 16 + 63) / 64; ++c) {
          const int i = lane + 64 * c;
          if (i < TILE_BYTES / 16) {
            ((u32x4_t *)sK)[i] = __builtin_nontemporal_load(ksrc + i);
            ((u32x4_t *)sV)[i] = __builtin_nontemporal_load(vsrc + i);
          }
        }
        wave_lds_fence();
      }

      // ---- q*d operands (B, lane = head r) and zero-point operands (A, any row) -----------------
      half8_t qdh[KK], qdl[KK], mk[KK];
#pragma unroll
      for (int kk = 0; kk < KK; ++kk)
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const uint8_t *blk = sK + (32 * kk + 8 * j + e) * BB;
          const float dd = (float)*(const _Float16 *)blk;
          mk[kk][e] = *(const _Float16 *)(blk + 2);
          _Float16 hi, lo;
          split_f16(qf[kk][e] * dd, hi, lo);
          qdh[kk][e] = hi;
          qdl[kk][e] = lo;
        }

      // ---- logits: two halves of 16 tokens (row m = r -> token 16*half + r) ---------------------
#pragma unroll
      for (int hf = 0; hf < 2; ++hf) {
        const int byte_off = 4 + ((16 * hf + r) * BITS) / 8;
#pragma unroll
        for (int kk = 0; kk < KK; ++kk) {
          const uint8_t *cp = sK + (32 * kk + 8 * j) * BB + byte_off;
          const half8_t a = make_half8(codes_to_half2(cp[0], cp[BB], mask_r), codes_to_half2(cp[2 * BB], cp[3 * BB], mask_r),
                                       codes_to_half2(cp[4 * BB], cp[5 * BB], mask_r), codes_to_half2(cp[6 * BB], cp[7 * BB], mask_r));
          s[hf] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, qdh[kk], s[hf], 0, 0, 0);
          s[hf] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, qdl[kk], s[hf], 0, 0, 0);
        }
      }
      // result register i belongs to token 16*half + 4j + i: undo that token's sub-byte shift
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float f = 1.0f / (float)(1 << ((i * BITS) % 8));
        s[0][i] *= f;
        s[1][i] *= f;
      }
      // zero-point term sum_ch m[ch] q[h][ch]: identical for every token row
      float4_t c0 = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
      for (int kk = 0; kk < KK; ++kk) {
        c0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(mk[kk], qh[kk], c0, 0, 0, 0);
        c0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(mk[kk], ql[kk], c0, 0, 0, 0);
      }
      s[0] = (s[0] + c0) * (1.0f / kOpScale);
      s[1] = (s[1] + c0) * (1.0f / kOpScale);
    } else {
      // ---- residual rows: [kv_heads, res_cap, D] F32 or F16 -------------------------------------
      const int ru = u - q_units;
      tok0 = kp.q_tokens + ru * kUnit;
      n_valid = min(kUnit, kp.res_tokens - ru * kUnit);
      if (shift_pending) {
#pragma unroll
        for (int a = 0; a < 2 * KK; ++a) o_acc[a] *= fv;
        shift_pending = false;
      }
      const int64_t rbase = (int64_t)b * kp.res_bs + (int64_t)kvh * kp.res_cap * D;
#pragma unroll
      for (int hf = 0; hf < 2; ++hf) {
        const int rt = ru * kUnit + min(16 * hf + r, n_valid - 1);
#pragma unroll
        for (int kk = 0; kk < KK; ++kk) {
          half8_t ah, al;
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            const int64_t idx = rbase + (int64_t)rt * D + 32 * kk + 8 * j + e;
            const float x = kp.res_f16 ? (float)((const _Float16 *)kp.res_k)[idx] : ((const float *)kp.res_k)[idx];
            _Float16 hi, lo;
            split_f16(x, hi, lo);
            ah[e] = hi;
            al[e] = lo;
          }
          s[hf] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ah, qh[kk], s[hf], 0, 0, 0);
          s[hf] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ah, ql[kk], s[hf], 0, 0, 0);
          s[hf] = __builtin_amdgcn_mfma_f32_16x16x32_f16(al, qh[kk], s[hf], 0, 0, 0);
        }
        s[hf] *= 1.0f / kOpScale;
      }
    }

    // ---- online softmax over the unit's 32 tokens; lane (j, h = r) owns tokens tok_of(j, e) ------
    float mt = kNegInf;
#pragma unroll
    for (int hf = 0; hf < 2; ++hf)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        if (16 * hf + 4 * j + i >= n_valid) s[hf][i] = kNegInf;
        mt = fmaxf(mt, s[hf][i]);  // a NaN logit propagates (the reference kernels have no guard)
      }
    if (p.scores && r < G) {
      float *srow = p.scores + (int64_t)b * p.score_bs + (int64_t)(kvh * G + r) * p.score_stride + tok0;
#pragma unroll
      for (int hf = 0; hf < 2; ++hf)
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (16 * hf + 4 * j + i < n_valid) srow[16 * hf + 4 * j + i] = s[hf][i] * kLn2;
    }
    mt = fmaxf(mt, __shfl_xor(mt, 16, 64));
    mt = fmaxf(mt, __shfl_xor(mt, 32, 64));
    const float m_new = fmaxf(m_run, mt);
    const float m_ref = (m_new == kNegInf) ? 0.0f : m_new;
    const float alpha = __builtin_amdgcn_exp2f(m_run - m_ref);
    m_run = m_new;
    half8_t pa;
    float lsum = 0.0f;  // f32 sum: the emitted probabilities are normalised by it
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float pw = __builtin_amdgcn_exp2f(s[e / 4][e % 4] - m_ref);  // NaN stays NaN
      lsum += pw;
      pa[e] = (_Float16)pw;
    }
    l_run = l_run * alpha + lsum;
    if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0) {
      float al[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) al[i] = __shfl(alpha, 4 * j + i, 64);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
#pragma unroll
        for (int a = 0; a < 2 * KK; ++a) o_acc[a][i] *= al[i];
        m_acc[i] *= al[i];
      }
    }

    // ---- output ----------------------------------------------------------------------------------
    if (quant) {
      const half8_t pa_s = pa * (_Float16)kOpScale;  // keeps small p*d out of the f16 subnormals
#pragma unroll
      for (int cb = 0; cb < KK; ++cb) {
        // A operand: p * d[token][cb] (lane = head r, k-slot e -> token tok_of(j, e))
        half8_t dv;
#pragma unroll
        for (int e = 0; e < 8; ++e) dv[e] = *(const _Float16 *)(sV + (tok_of(j, e) * KK + cb) * BB);
        const half8_t pd = pa_s * dv;
#pragma unroll
        for (int sub = 0; sub < 2; ++sub) {
          // B operand: codes of channel 32cb + 16sub + r for tokens tok_of(j, e)
          const int byte_off = cb * BB + 4 + ((16 * sub + r) * BITS) / 8;
          uint32_t bt[8];
#pragma unroll
          for (int e = 0; e < 8; ++e) bt[e] = sV[tok_of(j, e) * KK * BB + byte_off];
          const half8_t bc = make_half8(codes_to_half2(bt[0], bt[1], mask_r), codes_to_half2(bt[2], bt[3], mask_r),
                                        codes_to_half2(bt[4], bt[5], mask_r), codes_to_half2(bt[6], bt[7], mask_r));
          o_acc[2 * cb + sub] = __builtin_amdgcn_mfma_f32_16x16x32_f16(pd, bc, o_acc[2 * cb + sub], 0, 0, 0);
        }
      }
      // zero-point term: column n = cb holds sum_t p[h][t] m[t][cb]
      half8_t mv = {0, 0, 0, 0, 0, 0, 0, 0};
      if (r < KK) {
#pragma unroll
        for (int e = 0; e < 8; ++e) mv[e] = *(const _Float16 *)(sV + (tok_of(j, e) * KK + r) * BB + 2);
      }
      m_acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(pa, mv, m_acc, 0, 0, 0);
    } else {
      const int ru = u - q_units;
      const int64_t rbase = (int64_t)b * kp.res_bs + (int64_t)kvh * kp.res_cap * D;
#pragma unroll
      for (int cs = 0; cs < 2 * KK; ++cs) {
        half8_t bv;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const int rt = ru * kUnit + min(tok_of(j, e), n_valid - 1);
          const int64_t idx = rbase + (int64_t)rt * D + 16 * cs + r;
          bv[e] = kp.res_f16 ? ((const _Float16 *)kp.res_v)[idx] : (_Float16)((const float *)kp.res_v)[idx];
        }
        o_acc[cs] = __builtin_amdgcn_mfma_f32_16x16x32_f16(pa, bv, o_acc[cs], 0, 0, 0);
      }
    }
  }
  if (shift_pending) {
#pragma unroll
    for (int a = 0; a < 2 * KK; ++a) o_acc[a] *= fv;
  }

  // ---- merge: lane groups (row sum), then the 4 waves through LDS --------------------------------
  l_run += __shfl_xor(l_run, 16, 64);
  l_run += __shfl_xor(l_run, 32, 64);
  __syncthreads();  // every wave is done with its tile region
  float(*lds_acc)[16][D + 4] = (float(*)[16][D + 4]) smem;
  float(*lds_mt)[16][KK] = (float(*)[16][KK])(smem + 4 * 16 * (D + 4) * 4);
  float(*lds_m)[16] = (float(*)[16])(smem + 4 * 16 * (D + 4) * 4 + 4 * 16 * KK * 4);
  float(*lds_l)[16] = lds_m + 4;
  if (j == 0) {
    lds_m[wave][r] = m_run;
    lds_l[wave][r] = l_run;
  }
#pragma unroll
  for (int a = 0; a < 2 * KK; ++a)
#pragma unroll
    for (int i = 0; i < 4; ++i) lds_acc[wave][4 * j + i][16 * a + r] = o_acc[a][i];
  if (r < KK) {
#pragma unroll
    for (int i = 0; i < 4; ++i) lds_mt[wave][4 * j + i][r] = m_acc[i];
  }
  __syncthreads();

  for (int idx = threadIdx.x; idx < G * D; idx += 256) {
    const int g = idx / D, c = idx % D;
    const int h = kvh * G + g;
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
  const int pairs = p.n_heads_kv * batch;
  const int target_wgs = ctx->compute_units * 4;
  // at least one unit per wave
  const int max_splits = (kp.units_total + 3) / 4;
  int nsplit = std::max(1, std::min({(target_wgs + pairs - 1) / pairs, max_splits, kMaxSplits}));
  kp.units_per_split = (kp.units_total + nsplit - 1) / nsplit;
  nsplit = (kp.units_total + kp.units_per_split - 1) / kp.units_per_split;
  p.nsplit = nsplit;
  p.direct = 0;
  const size_t n_part = (size_t)batch * p.n_heads_q * nsplit;
  const size_t ml_bytes = (n_part * 2 * sizeof(float) + 255) / 256 * 256;
  int rc = argus_ws_reserve(ctx, ml_bytes + n_part * D * sizeof(float));
  if (rc != ARGUS_HIP_OK) return rc;
  p.ws_ml = ctx->ws;
  p.ws_o = (float *)((char *)ctx->ws + ml_bytes);
  {
    KernelTimer timer(ctx, stream);
    hipLaunchKernelGGL((kivi_mfma_kernel<BITS, D>), dim3(nsplit, p.n_heads_kv, batch), dim3(256), 0, stream, kp);
  }
  ARGUS_HIP_CHECK(ctx, hipGetLastError());
  hipLaunchKernelGGL((decode_combine_kernel<NoFallback, D>), dim3(p.n_heads_q, batch), dim3(256), 0, stream, p);
  ARGUS_HIP_CHECK(ctx, hipGetLastError());
  return ARGUS_HIP_OK;
}

template <int BITS>
int launch_dim(argus_hip_ctx *ctx, KiviParams &kp, int batch, hipStream_t stream) {
  return kp.head_dim == 64 ? launch<BITS, 64>(ctx, kp, batch, stream) : launch<BITS, 128>(ctx, kp, batch, stream);
}

}  // namespace

bool kivi_mfma_supported(const KiviParams &kp) {
  const DecodeParams &p = kp.d;
  if (kp.head_dim != 64 && kp.head_dim != 128) return false;
  if (p.group > 16 || p.softcap > 0.0f) return false;
  // tiles are copied as 16-byte vectors
  if ((((uintptr_t)kp.qk | (uintptr_t)kp.qv) & 15) || (kp.qk_bs & 15) || (kp.qv_bs & 15)) return false;
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
