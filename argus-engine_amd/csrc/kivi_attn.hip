// KIVI fused dequant + decode attention (Q2 / Q4 / Q8 blocks + residual window), plus the
// residual-ring append and the on-device quantise-at-flush.
//
// Stands in for CudaQuantAttnBackend::{attention_gen_quant, gather_update_quant}
// (crates/argus-extension-api/src/lib.rs:3087-3104); arithmetic of
// crates/techniques/kivi/src/kivi_attn.cu:34-573 (dequant `code*d + m`, quantised tokens first,
// then the residual rows) over the block layouts of
// engine/src/kv/quant_window_cache.rs:919-946 (K per channel: flush -> head -> group -> channel;
// V per token: flush -> head -> token -> d/32 blocks) and the codec of
// crates/argus-kv-codec/src/lib.rs:26-203.
//
// Structure: the same split-KV scheme as the F16 decode.  A workgroup owns one KV head and a
// range of 32-token units.  For a quantised unit the K tile (head_dim blocks, contiguous) and
// the V tile (32 tokens x head_dim/32 blocks, contiguous) are copied into LDS with coalesced
// dword loads; logits are then formed with lanes = tokens (each thread walks a slice of the
// channels of its token, reading its code byte and the block header from LDS), an online
// softmax step runs over the 32 tokens, and the V phase runs with lanes = channels.  All GQA
// query heads of the KV head share the single pass over the blocks.
#include "kivi_common.hpp"

#include <algorithm>
#include <cstdlib>
#include <cstring>

namespace {

using namespace argus_decode;
using namespace argus_kivi;

template <int BITS>
__device__ __forceinline__ float kivi_code(const uint8_t *qs, int i) {
  if constexpr (BITS == 8) return (float)qs[i];
  if constexpr (BITS == 4) return (float)((qs[i >> 1] >> ((i & 1) * 4)) & 0x0F);
  return (float)((qs[i >> 2] >> ((i & 3) * 2)) & 0x03);
}

__device__ __forceinline__ float load_res(const void *base, int64_t i, int f16) {
  return f16 ? (float)((const _Float16 *)base)[i] : ((const float *)base)[i];
}

template <int BITS, int GT>
__global__ __launch_bounds__(256) void kivi_split_kernel(const KiviParams kp) {
  constexpr int BB = 4 + 32 * BITS / 8;  // block bytes
  constexpr int MAXD = 256;
  const DecodeParams &p = kp.d;
  const int D = kp.head_dim;
  // a GQA group wider than the head tile: several workgroups per KV head, GT heads each
  const int split = blockIdx.x, kvh = blockIdx.y / p.head_chunks, b = blockIdx.z;
  const int hbase = kvh * p.group + GT * (blockIdx.y % p.head_chunks);
  const int gcount = min(GT, p.group - GT * (int)(blockIdx.y % p.head_chunks));
  const int tid = threadIdx.x;
  const uint8_t *qk_b = kp.qk + (int64_t)b * kp.qk_bs;
  const uint8_t *qv_b = kp.qv + (int64_t)b * kp.qv_bs;
  const int64_t res_off = (int64_t)b * kp.res_bs;
  const int gpf = kp.res_cap / kUnit;   // K groups per flush
  const int bpt = D / kUnit;            // V blocks per token
  const int q_units = kp.q_tokens / kUnit;

  __shared__ __attribute__((aligned(16))) uint8_t sh_k[MAXD * BB];
  __shared__ __attribute__((aligned(16))) uint8_t sh_v[kUnit * (MAXD / kUnit) * BB];
  __shared__ float sh_q[MAXD][GT];        // q[ch][g] * scale
  __shared__ float sh_part[8][kUnit][GT]; // partial logits per channel slice
  __shared__ float sh_p[kUnit][GT];       // unit probabilities (relative to the running max)
  __shared__ float sh_alpha[GT], sh_m[GT], sh_l[GT];

  for (int i = tid; i < D * GT; i += 256) {
    const int ch = i / GT, g = i % GT;
    const int h = hbase + min(g, gcount - 1);
    sh_q[ch][g] = p.q[(int64_t)b * p.q_bs + (int64_t)h * D + ch] * p.scale;
  }
  if (tid < GT) {
    sh_m[tid] = kNegInf;
    sh_l[tid] = 0.0f;
  }

  // V-phase ownership: thread -> (channel c, token part tp); parts split the unit's 32 tokens.
  const int vparts = 256 / D;                 // 4, 2, 1 for D = 64, 128, 256
  const int vc = tid % D, vtp = tid / D;
  const int vtok = kUnit / vparts;
  float acc[GT];
#pragma unroll
  for (int g = 0; g < GT; ++g) acc[g] = 0.0f;

  // K-phase ownership: thread -> (token t, channel part cp); 8 parts split the channels.
  const int kt = tid % kUnit, kcp = tid / kUnit;
  const int kch = D / 8;
  const bool use_cap = p.softcap > 0.0f;
  const float inv_cap = use_cap ? 1.0f / p.softcap : 0.0f;

  const int u_begin = split * kp.units_per_split;
  const int u_end = min(kp.units_total, u_begin + kp.units_per_split);
  for (int u = u_begin; u < u_end; ++u) {
    const bool quant = u < q_units;
    const int tok0 = quant ? u * kUnit : kp.q_tokens + (u - q_units) * kUnit;  // logical token of row 0
    const int n_valid = quant ? kUnit : min(kUnit, kp.res_tokens - (u - q_units) * kUnit);
    __syncthreads();  // previous unit's LDS tiles are no longer read
    if (quant) {
      // K tile: blocks (flush, kvh, gif, ch = 0..D) are contiguous (kivi_attn.cu:256-262).
      const int flush = u / gpf, gif = u % gpf;
      const int64_t kblk = ((int64_t)flush * p.n_heads_kv * gpf + (int64_t)kvh * gpf + gif) * D;
      const uint32_t *ksrc = (const uint32_t *)(qk_b + kblk * BB);
      for (int i = tid; i < D * BB / 4; i += 256) ((uint32_t *)sh_k)[i] = __builtin_nontemporal_load(ksrc + i);
      // V tile: blocks (flush, kvh, tif, b) with tif = 32 consecutive tokens (kivi_attn.cu:357-361).
      const int tif0 = (u * kUnit) % kp.res_cap;
      const int64_t vblk = (((int64_t)flush * p.n_heads_kv + kvh) * kp.res_cap + tif0) * bpt;
      const uint32_t *vsrc = (const uint32_t *)(qv_b + vblk * BB);
      for (int i = tid; i < kUnit * bpt * BB / 4; i += 256) ((uint32_t *)sh_v)[i] = __builtin_nontemporal_load(vsrc + i);
    }
    __syncthreads();

    // ---- logits: thread (token kt, channel part kcp) ---------------------------------------
    {
      float part[GT];
#pragma unroll
      for (int g = 0; g < GT; ++g) part[g] = 0.0f;
      if (quant) {
        for (int c = 0; c < kch; ++c) {
          const int ch = kcp * kch + c;
          const uint8_t *blk = sh_k + ch * BB;
          const float dd = (float)*(const _Float16 *)blk;
          const float mm = (float)*(const _Float16 *)(blk + 2);
          const float x = kivi_code<BITS>(blk + 4, kt) * dd + mm;
#pragma unroll
          for (int g = 0; g < GT; ++g) part[g] = fmaf(sh_q[ch][g], x, part[g]);
        }
      } else if (kt < n_valid) {
        const int rt = (u - q_units) * kUnit + kt;
        const int64_t rbase = res_off + ((int64_t)kvh * kp.res_cap + rt) * D + kcp * kch;
        for (int c = 0; c < kch; ++c) {
          const float x = load_res(kp.res_k, rbase + c, kp.res_f16);
#pragma unroll
          for (int g = 0; g < GT; ++g) part[g] = fmaf(sh_q[kcp * kch + c][g], x, part[g]);
        }
      }
#pragma unroll
      for (int g = 0; g < GT; ++g) sh_part[kcp][kt][g] = part[g];
    }
    __syncthreads();

    // ---- online softmax over the unit: thread (token t, head g), tid < 32 * GT -------------
    if (tid < kUnit * GT) {
      const int g = tid / kUnit, t = tid % kUnit;
      float sv = 0.0f;
#pragma unroll
      for (int cp = 0; cp < 8; ++cp) sv += sh_part[cp][t][g];
      if (use_cap) {
        const float capped = softcap_tanh(sv, p.softcap, inv_cap);
        sv = (sv != sv) ? sv : capped;
      }
      if (t >= n_valid) sv = kNegInf;
      if (p.scores && g < gcount && t < n_valid)
        p.scores[(int64_t)b * p.score_bs + (int64_t)(hbase + g) * p.score_stride + tok0 + t] = sv;
      const float m_old = sh_m[g];
      const float m_new = fmaxf(m_old, group_allreduce_max<32>(sv));
      const float m_ref = (m_new == kNegInf) ? 0.0f : m_new;
      const float pw = __expf(sv - m_ref);
      const float lsum = group_allreduce_sum<32>(pw);
      sh_p[t][g] = pw;
      if (t == 0) {
        const float alpha = __expf(m_old - m_ref);
        sh_alpha[g] = alpha;
        sh_m[g] = m_new;
        sh_l[g] = sh_l[g] * alpha + lsum;
      }
    }
    __syncthreads();

    // ---- V phase: thread (channel vc, token part vtp) ---------------------------------------
#pragma unroll
    for (int g = 0; g < GT; ++g) acc[g] *= sh_alpha[g];
    if (quant) {
      const int b = vc / kUnit, ci = vc % kUnit;
      for (int tt = 0; tt < vtok; ++tt) {
        const int t = vtp * vtok + tt;
        const uint8_t *blk = sh_v + (t * bpt + b) * BB;
        const float dd = (float)*(const _Float16 *)blk;
        const float mm = (float)*(const _Float16 *)(blk + 2);
        const float x = kivi_code<BITS>(blk + 4, ci) * dd + mm;
#pragma unroll
        for (int g = 0; g < GT; ++g) acc[g] = fmaf(sh_p[t][g], x, acc[g]);
      }
    } else {
      for (int tt = 0; tt < vtok; ++tt) {
        const int t = vtp * vtok + tt;
        if (t < n_valid) {
          const int rt = (u - q_units) * kUnit + t;
          const float x = load_res(kp.res_v, res_off + ((int64_t)kvh * kp.res_cap + rt) * D + vc, kp.res_f16);
#pragma unroll
          for (int g = 0; g < GT; ++g) acc[g] = fmaf(sh_p[t][g], x, acc[g]);
        }
      }
    }
  }

  // ---- reduce the token parts, write the split partial --------------------------------------
  __syncthreads();
  float *red = (float *)sh_part;  // reuse: [vparts][GT][D] floats <= 8*32*GT
  if (vparts > 1) {
#pragma unroll
    for (int g = 0; g < GT; ++g) red[(vtp * GT + g) * D + vc] = acc[g];
    __syncthreads();
  }
  if (vtp == 0) {
#pragma unroll
    for (int g = 0; g < GT; ++g) {
      if (g >= gcount) continue;
      float o = acc[g];
      for (int tp = 1; tp < vparts; ++tp) o += red[(tp * GT + g) * D + vc];
      const int h = hbase + g;
      const int64_t pidx = ((int64_t)b * p.n_heads_q + h) * p.nsplit + split;
      p.ws_o[pidx * D + vc] = o;
      if (vc == 0) {
        p.ws_ml[pidx * 2 + 0] = sh_m[g];
        p.ws_ml[pidx * 2 + 1] = sh_l[g];
      }
    }
  }
}

// gather_update_quant: residual[h, res_pos + s, :] = input[s, h, :] (kivi_q2.cu:117-138).
__global__ __launch_bounds__(256) void kivi_gather_update_kernel(const float *__restrict__ input,
                                                                 float *__restrict__ residual, int kv_heads,
                                                                 int res_cap, int head_dim, int seq_len, int res_pos) {
  const int vec = head_dim / 4;
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= (int64_t)seq_len * kv_heads * vec) return;
  const int c = (int)(i % vec) * 4;
  const int64_t row = i / vec;
  const int h = (int)(row % kv_heads);
  const int64_t s = row / kv_heads;
  *(float4_t *)(residual + ((int64_t)h * res_cap + res_pos + s) * head_dim + c) =
      *(const float4_t *)(input + row * head_dim + c);
}

// ---- quantise-at-flush -------------------------------------------------------------------------
// One thread quantises one 32-value block with the exact operation order of
// BlockQ2_0 / BlockKVQ4 / BlockKVQ8::quantize (crates/argus-kv-codec/src/lib.rs:36-59, 125-145,
// 175-192): f32 min/max fold, d = range / (2^b - 1), id = 1/d (0 when d == 0),
// q = round_half_away((x - min) * id) clamped, d and min stored as RNE f16.  The explicit
// *_rn intrinsics keep the compiler from contracting or reassociating the arithmetic.
template <int BITS>
__device__ __forceinline__ void quantize_block(const float (&x)[32], uint8_t *dst) {
  float mn = __builtin_huge_valf(), mx = -__builtin_huge_valf();
#pragma unroll
  for (int i = 0; i < 32; ++i) {
    mn = fminf(mn, x[i]);
    mx = fmaxf(mx, x[i]);
  }
  constexpr float hi = (float)((1 << BITS) - 1);
  const float d = __fdiv_rn(__fsub_rn(mx, mn), hi);
  const float id = (d == 0.0f) ? 0.0f : __fdiv_rn(1.0f, d);
  uint32_t words[1 + 8 * BITS / 8];
  const _Float16 dh = (_Float16)d, mh = (_Float16)mn;
  words[0] = (uint32_t)__builtin_bit_cast(uint16_t, dh) | ((uint32_t)__builtin_bit_cast(uint16_t, mh) << 16);
#pragma unroll
  for (int w = 0; w < 8 * BITS / 8; ++w) words[1 + w] = 0;
#pragma unroll
  for (int i = 0; i < 32; ++i) {
    float r = roundf(__fmul_rn(__fsub_rn(x[i], mn), id));
    r = fminf(fmaxf(r, 0.0f), hi);  // NaN -> 0 like the saturating `as u8`
    const uint32_t c = (uint32_t)r;
    const int bit = i * BITS;
    words[1 + bit / 32] |= c << (bit % 32);
  }
#pragma unroll
  for (int w = 0; w < 1 + 8 * BITS / 8; ++w) ((uint32_t *)dst)[w] = words[w];
}

template <int BITS>
__global__ __launch_bounds__(128) void kivi_flush_k_kernel(const float *__restrict__ res_k, uint8_t *__restrict__ qk,
                                                           int kv_heads, int res_cap, int head_dim, int n_groups,
                                                           int64_t block_start, int out_gpf) {
  constexpr int BB = 4 + 32 * BITS / 8;
  // block order h -> group -> ch (quant_window_cache.rs:919-930); thread per block, ch fastest so
  // the 32 strided row reads of a wave are coalesced across channels.  out_gpf: the groups are laid
  // out as consecutive flushes of that many groups each (flush -> h -> group in flush -> ch).
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= (int64_t)kv_heads * n_groups * head_dim) return;
  const int ch = (int)(i % head_dim);
  const int g = (int)((i / head_dim) % n_groups);
  const int h = (int)(i / ((int64_t)head_dim * n_groups));
  float x[32];
#pragma unroll
  for (int t = 0; t < 32; ++t) x[t] = res_k[((int64_t)h * res_cap + g * 32 + t) * head_dim + ch];
  const int64_t o = (((int64_t)(g / out_gpf) * kv_heads + h) * out_gpf + g % out_gpf) * head_dim + ch;
  quantize_block<BITS>(x, qk + (block_start + o) * BB);
}

template <int BITS>
__global__ __launch_bounds__(128) void kivi_flush_v_kernel(const float *__restrict__ res_v, uint8_t *__restrict__ qv,
                                                           int kv_heads, int res_cap, int head_dim, int flush_tokens,
                                                           int64_t block_start, int out_cap) {
  constexpr int BB = 4 + 32 * BITS / 8;
  // block order h -> t -> b (quant_window_cache.rs:932-946), in flushes of out_cap tokens
  const int bpt = head_dim / 32;
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= (int64_t)kv_heads * flush_tokens * bpt) return;
  const int b = (int)(i % bpt);
  const int t = (int)((i / bpt) % flush_tokens);
  const int h = (int)(i / ((int64_t)bpt * flush_tokens));
  const float4_t *src = (const float4_t *)(res_v + ((int64_t)h * res_cap + t) * head_dim + b * 32);
  float x[32];
#pragma unroll
  for (int v = 0; v < 8; ++v) {
    const float4_t f = src[v];
    x[4 * v] = f[0];
    x[4 * v + 1] = f[1];
    x[4 * v + 2] = f[2];
    x[4 * v + 3] = f[3];
  }
  const int64_t o = (((int64_t)(t / out_cap) * kv_heads + h) * out_cap + t % out_cap) * bpt + b;
  quantize_block<BITS>(x, qv + (block_start + o) * BB);
}

// ---- bit-width transition ------------------------------------------------------------------------
// QuantizedRecentWindowCache::transition_bits between two quantised widths
// (engine/src/kv/quant_window_cache.rs:1308-1372): every block is dequantised to 32 f32 values
// (`q * d + m`, crates/argus-kv-codec/src/lib.rs:61-72: the product of a code and an f16 scale is
// exact in f32, so the sum rounds once) and quantised again at the new width; block count and order
// stay.  One thread per block.
template <int OLD, int NEW>
__global__ __launch_bounds__(128) void kivi_requant_kernel(const uint8_t *__restrict__ src, uint8_t *__restrict__ dst, int64_t n_blocks) {
  constexpr int OB = 4 + 32 * OLD / 8, NB = 4 + 32 * NEW / 8;
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n_blocks) return;
  const uint32_t *w = (const uint32_t *)(src + i * OB);  // block sizes are multiples of 4
  uint32_t words[OB / 4];
#pragma unroll
  for (int k = 0; k < OB / 4; ++k) words[k] = w[k];
  const float d = (float)__builtin_bit_cast(_Float16, (uint16_t)(words[0] & 0xffffu));
  const float m = (float)__builtin_bit_cast(_Float16, (uint16_t)(words[0] >> 16));
  float x[32];
#pragma unroll
  for (int e = 0; e < 32; ++e) {
    const int bit = e * OLD;
    const uint32_t c = (words[1 + bit / 32] >> (bit % 32)) & ((1u << OLD) - 1u);
    x[e] = __fadd_rn(__fmul_rn((float)c, d), m);
  }
  quantize_block<NEW>(x, dst + i * NB);
}

template <int BITS>
int launch_kivi(argus_hip_ctx *ctx, KiviParams &kp, int batch, hipStream_t stream) {
  // ARGUS_HIP_KIVI=valu (read when the context is created) keeps the vector-ALU kernel for A/B measurements.
  const bool force_valu = ctx->env.kivi_valu;
  if (!force_valu && kivi_mfma_supported(kp)) return launch_kivi_mfma(ctx, kp, BITS, batch, stream);
  DecodeParams &p = kp.d;
  const int D = kp.head_dim;
  const int target_wgs = ctx->compute_units * 4;
  p.head_chunks = (p.group + 7) / 8;  // head tile of the widest instantiation
  const int pairs = p.n_heads_kv * p.head_chunks * batch;
  int nsplit = std::max(1, std::min({(target_wgs + pairs - 1) / pairs, kp.units_total, kMaxSplits}));
  kp.units_per_split = (kp.units_total + nsplit - 1) / nsplit;
  nsplit = (kp.units_total + kp.units_per_split - 1) / kp.units_per_split;
  p.nsplit = nsplit;
  p.direct = 0;
  const int rc = reserve_partials(ctx, p, batch, D);
  if (rc != ARGUS_HIP_OK) return rc;
  ctx->plan = argus_hip_decode_plan{nsplit, kp.units_per_split * kUnit, 0, 0, 2, 4, 0};

  dim3 grid(nsplit, p.n_heads_kv * p.head_chunks, batch);
  KernelTimer timer(ctx, stream);
  if (p.group <= 1) hipLaunchKernelGGL((kivi_split_kernel<BITS, 1>), grid, dim3(256), 0, stream, kp);
  else if (p.group <= 2) hipLaunchKernelGGL((kivi_split_kernel<BITS, 2>), grid, dim3(256), 0, stream, kp);
  else if (p.group <= 4) hipLaunchKernelGGL((kivi_split_kernel<BITS, 4>), grid, dim3(256), 0, stream, kp);
  else hipLaunchKernelGGL((kivi_split_kernel<BITS, 8>), grid, dim3(256), 0, stream, kp);
  timer.mark();
  ARGUS_HIP_CHECK(ctx, hipGetLastError());
  switch (D) {
    case 64: hipLaunchKernelGGL((decode_combine_kernel<NoFallback, 64>), combine_grid(p, batch), dim3(256), 0, stream, p); break;
    case 128: hipLaunchKernelGGL((decode_combine_kernel<NoFallback, 128>), combine_grid(p, batch), dim3(256), 0, stream, p); break;
    default: hipLaunchKernelGGL((decode_combine_kernel<NoFallback, 256>), combine_grid(p, batch), dim3(256), 0, stream, p); break;
  }
  ARGUS_HIP_CHECK(ctx, hipGetLastError());
  return ARGUS_HIP_OK;
}

bool bits_ok(uint8_t bits) { return bits == 2 || bits == 4 || bits == 8; }

}  // namespace

ARGUS_API int argus_hip_has_quant_attn_kernel(const argus_hip_ctx *ctx, uint8_t bits) {
  return (ctx && bits_ok(bits)) ? 1 : 0;
}

ARGUS_API int argus_hip_attention_gen_quant_ex(argus_hip_ctx *ctx, const argus_hip_quant_attn_args *a,
                                               const argus_hip_quant_attn_ext *ext) {
  if (!ctx || !a) return ARGUS_HIP_ERR_INVALID;
  // Error behaviour of KiviCudaBackend::attention_inner (gpu_kivi_cuda.rs:126-140).
  if (!bits_ok(a->bits)) return argus_fail(ctx, ARGUS_HIP_ERR_UNSUPPORTED, "unsupported KIVI bits: %d", (int)a->bits);
  if (a->num_heads_q == 0 || a->num_heads_kv == 0 || a->num_heads_q % a->num_heads_kv)
    return argus_fail(ctx, ARGUS_HIP_ERR_INVALID, "attention_gen_quant: heads %zu/%zu", a->num_heads_q, a->num_heads_kv);
  const size_t D = a->head_dim;
  if (D != 64 && D != 128 && D != 256)
    return argus_fail(ctx, ARGUS_HIP_ERR_UNSUPPORTED, "attention_gen_quant: head_dim %zu not in {64,128,256}", D);
  if (a->res_cap == 0 || a->res_cap % kUnit || a->q_tokens % kUnit || a->res_tokens > a->res_cap)
    return argus_fail(ctx, ARGUS_HIP_ERR_INVALID, "attention_gen_quant: q_tokens %zu res_tokens %zu res_cap %zu",
                      a->q_tokens, a->res_tokens, a->res_cap);
  const size_t total = a->q_tokens + a->res_tokens;
  if (total == 0) return argus_fail(ctx, ARGUS_HIP_ERR_INVALID, "attention_gen_quant: no tokens");
  if (!a->q_mem || !a->out_mem || (a->q_tokens && (!a->qk_mem || !a->qv_mem)) ||
      (a->res_tokens && (!a->res_k_mem || !a->res_v_mem)))
    return argus_fail(ctx, ARGUS_HIP_ERR_INVALID, "attention_gen_quant: null buffer");
  if ((a->qk_mem | a->qv_mem) & 3)
    return argus_fail(ctx, ARGUS_HIP_ERR_INVALID, "attention_gen_quant: block streams must be 4-byte aligned");
  if (a->out_mem & 15) return argus_fail(ctx, ARGUS_HIP_ERR_INVALID, "attention_gen_quant: out must be 16-byte aligned");

  hipStream_t stream = (hipStream_t)a->stream;
  const bool want_host = a->scores_out != nullptr && a->scores_len > 0;
  const bool want_dev = ext && ext->scores_dev != 0;
  // score_stride: scores_len / num_heads_q on the host path (gpu_kivi_cuda.rs:143-149).
  size_t stride = want_dev ? ext->score_stride : (want_host ? a->scores_len / a->num_heads_q : 0);
  if ((want_host || want_dev) && stride < total)
    return argus_fail(ctx, ARGUS_HIP_ERR_INVALID, "attention_gen_quant: score stride %zu < tokens %zu", stride, total);

  float *scores_dev = want_dev ? (float *)ext->scores_dev : nullptr;
  float *transient = nullptr;
  if (want_host && !want_dev) {
    // Transient device score buffer, freed before return (gpu_kivi_cuda.rs:147-153, 217-222).
    if (hipMalloc((void **)&transient, a->num_heads_q * stride * sizeof(float)) != hipSuccess) {
      (void)hipGetLastError();
      return argus_fail(ctx, ARGUS_HIP_ERR_NOMEM, "attention_gen_quant: score buffer allocation failed");
    }
    scores_dev = transient;
  }

  KiviParams kp{};
  DecodeParams &p = kp.d;
  p.q = (const float *)a->q_mem;
  p.out = (float *)a->out_mem;
  p.scores = scores_dev;
  p.n_heads_q = (int32_t)a->num_heads_q;
  p.n_heads_kv = (int32_t)a->num_heads_kv;
  p.group = p.n_heads_q / p.n_heads_kv;
  p.len = (int32_t)total;
  p.score_stride = (int32_t)stride;
  p.q_bs = p.out_bs = (int64_t)a->num_heads_q * D;
  p.score_bs = (int64_t)a->num_heads_q * stride;
  if (ext && ext->score_stats_dev) {
    if (!want_dev || want_host)
      return argus_fail(ctx, ARGUS_HIP_ERR_INVALID, "attention_gen_quant: score_stats_dev goes with scores_dev (and no host slice)");
    p.score_stats = (float *)ext->score_stats_dev;
    p.stats_bs = (int64_t)a->num_heads_q * 2;
  }
  p.scale = a->scale;
  p.softcap = ext ? ext->softcap : 0.0f;
  kp.qk = (const uint8_t *)a->qk_mem;
  kp.qv = (const uint8_t *)a->qv_mem;
  kp.res_k = (const void *)a->res_k_mem;
  kp.res_v = (const void *)a->res_v_mem;
  kp.head_dim = (int32_t)D;
  kp.q_tokens = (int32_t)a->q_tokens;
  kp.res_tokens = (int32_t)a->res_tokens;
  kp.res_cap = (int32_t)a->res_cap;
  kp.res_f16 = (ext && ext->res_dtype == ARGUS_HIP_F16) ? 1 : 0;
  kp.units_total = (int32_t)(a->q_tokens / kUnit + (a->res_tokens + kUnit - 1) / kUnit);
  const int batch = (ext && ext->batch > 1) ? ext->batch : 1;
  if (batch > 1) {
    if (want_host) return argus_fail(ctx, ARGUS_HIP_ERR_UNSUPPORTED, "attention_gen_quant: host score read-back is single-sequence");
    if (batch > 65535) return argus_fail(ctx, ARGUS_HIP_ERR_UNSUPPORTED, "attention_gen_quant: batch beyond grid limits");
    if ((ext->block_batch_stride_bytes & 3) || (a->q_tokens && ext->block_batch_stride_bytes == 0) ||
        (a->res_tokens && ext->res_batch_stride == 0))
      return argus_fail(ctx, ARGUS_HIP_ERR_INVALID, "attention_gen_quant: batch strides");
    kp.qk_bs = kp.qv_bs = ext->block_batch_stride_bytes;
    kp.res_bs = ext->res_batch_stride;
    p.score_bs = ext->score_batch_stride ? ext->score_batch_stride : (int64_t)a->num_heads_q * stride;
  }

  int rc;
  switch (a->bits) {
    case 2: rc = launch_kivi<2>(ctx, kp, batch, stream); break;
    case 4: rc = launch_kivi<4>(ctx, kp, batch, stream); break;
    default: rc = launch_kivi<8>(ctx, kp, batch, stream); break;
  }
  if (rc == ARGUS_HIP_OK && want_host) {
    // Blocking read-back into the host slice (gpu_kivi_cuda.rs:204-212).
    hipError_t e = hipSuccess;
    if (want_dev && stride * a->num_heads_q > a->scores_len) {
      rc = argus_fail(ctx, ARGUS_HIP_ERR_INVALID, "attention_gen_quant: host score slice too small");
    } else {
      e = hipMemcpyAsync(a->scores_out, scores_dev, a->num_heads_q * stride * sizeof(float), hipMemcpyDeviceToHost, stream);
      if (e == hipSuccess) e = hipStreamSynchronize(stream);
      if (e != hipSuccess) rc = argus_fail(ctx, ARGUS_HIP_ERR_RUNTIME, "score read-back: %s", hipGetErrorString(e));
    }
  }
  if (transient) {
    if (rc != ARGUS_HIP_OK) (void)hipStreamSynchronize(stream);
    (void)hipFree(transient);
  }
  return rc;
}

ARGUS_API int argus_hip_attention_gen_quant(argus_hip_ctx *ctx, const argus_hip_quant_attn_args *a) {
  return argus_hip_attention_gen_quant_ex(ctx, a, nullptr);
}

ARGUS_API int argus_hip_gather_update_quant(argus_hip_ctx *ctx, const argus_hip_quant_gather_args *a) {
  if (!ctx || !a) return ARGUS_HIP_ERR_INVALID;
  if (!a->input_mem || !a->residual_mem) return argus_fail(ctx, ARGUS_HIP_ERR_INVALID, "gather_update_quant: null buffer");
  if (a->head_dim == 0 || a->head_dim % 4 || a->kv_heads == 0 || a->res_pos + a->seq_len > a->res_cap)
    return argus_fail(ctx, ARGUS_HIP_ERR_INVALID, "gather_update_quant: res_pos %zu + seq_len %zu > res_cap %zu",
                      a->res_pos, a->seq_len, a->res_cap);
  if (a->seq_len == 0) return ARGUS_HIP_OK;
  const int64_t total = (int64_t)a->seq_len * a->kv_heads * (a->head_dim / 4);
  hipLaunchKernelGGL(kivi_gather_update_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0,
                     (hipStream_t)a->stream, (const float *)a->input_mem, (float *)a->residual_mem, (int)a->kv_heads,
                     (int)a->res_cap, (int)a->head_dim, (int)a->seq_len, (int)a->res_pos);
  ARGUS_HIP_CHECK(ctx, hipGetLastError());
  return ARGUS_HIP_OK;
}

ARGUS_API int argus_hip_quant_flush(argus_hip_ctx *ctx, const argus_hip_quant_flush_args *a) {
  if (!ctx || !a) return ARGUS_HIP_ERR_INVALID;
  if (!bits_ok(a->bits)) return argus_fail(ctx, ARGUS_HIP_ERR_UNSUPPORTED, "unsupported KIVI bits: %d", (int)a->bits);
  if (!a->res_k_mem || !a->res_v_mem || !a->qk_mem || !a->qv_mem)
    return argus_fail(ctx, ARGUS_HIP_ERR_INVALID, "quant_flush: null buffer");
  if (a->head_dim == 0 || a->head_dim % kUnit || a->flush_tokens % kUnit || a->flush_tokens > a->res_cap || a->kv_heads == 0)
    return argus_fail(ctx, ARGUS_HIP_ERR_INVALID, "quant_flush: head_dim %zu flush_tokens %zu res_cap %zu", a->head_dim,
                      a->flush_tokens, a->res_cap);
  if ((a->qk_mem | a->qv_mem) & 3 || (a->res_v_mem & 15))
    return argus_fail(ctx, ARGUS_HIP_ERR_INVALID, "quant_flush: misaligned buffer");
  if (a->out_res_cap && (a->out_res_cap % kUnit || a->flush_tokens % a->out_res_cap))
    return argus_fail(ctx, ARGUS_HIP_ERR_INVALID, "quant_flush: out_res_cap %zu does not divide flush_tokens %zu into whole groups",
                      a->out_res_cap, a->flush_tokens);
  if (a->flush_tokens == 0) return ARGUS_HIP_OK;
  hipStream_t stream = (hipStream_t)a->stream;
  const int n_groups = (int)(a->flush_tokens / kUnit);
  const int out_cap = (int)(a->out_res_cap ? a->out_res_cap : a->flush_tokens);
  const int64_t nk = (int64_t)a->kv_heads * n_groups * a->head_dim;
  const int64_t nv = (int64_t)a->kv_heads * a->flush_tokens * (a->head_dim / kUnit);
  const dim3 gk((unsigned)((nk + 127) / 128)), gv((unsigned)((nv + 127) / 128));
#define ARGUS_FLUSH(B)                                                                                              \
  hipLaunchKernelGGL((kivi_flush_k_kernel<B>), gk, dim3(128), 0, stream, (const float *)a->res_k_mem,               \
                     (uint8_t *)a->qk_mem, (int)a->kv_heads, (int)a->res_cap, (int)a->head_dim, n_groups,           \
                     (int64_t)a->k_block_start, out_cap / kUnit);                                                   \
  hipLaunchKernelGGL((kivi_flush_v_kernel<B>), gv, dim3(128), 0, stream, (const float *)a->res_v_mem,               \
                     (uint8_t *)a->qv_mem, (int)a->kv_heads, (int)a->res_cap, (int)a->head_dim, (int)a->flush_tokens, \
                     (int64_t)a->v_block_start, out_cap)
  switch (a->bits) {
    case 2: ARGUS_FLUSH(2); break;
    case 4: ARGUS_FLUSH(4); break;
    default: ARGUS_FLUSH(8); break;
  }
#undef ARGUS_FLUSH
  ARGUS_HIP_CHECK(ctx, hipGetLastError());
  return ARGUS_HIP_OK;
}

ARGUS_API int argus_hip_quant_requant(argus_hip_ctx *ctx, const argus_hip_quant_requant_args *a) {
  if (!ctx || !a) return ARGUS_HIP_ERR_INVALID;
  if (!bits_ok(a->old_bits) || !bits_ok(a->new_bits))
    return argus_fail(ctx, ARGUS_HIP_ERR_UNSUPPORTED, "quant_requant: bits %d -> %d", (int)a->old_bits, (int)a->new_bits);
  if (a->n_blocks == 0) return ARGUS_HIP_OK;
  if (!a->src_mem || !a->dst_mem || ((a->src_mem | a->dst_mem) & 3))
    return argus_fail(ctx, ARGUS_HIP_ERR_INVALID, "quant_requant: null or misaligned block stream");
  const uint64_t ob = 4 + 32 * (uint64_t)a->old_bits / 8, nb = 4 + 32 * (uint64_t)a->new_bits / 8;
  if (a->src_mem < a->dst_mem + a->n_blocks * nb && a->dst_mem < a->src_mem + a->n_blocks * ob)
    return argus_fail(ctx, ARGUS_HIP_ERR_INVALID, "quant_requant: source and destination streams overlap");
  hipStream_t stream = (hipStream_t)a->stream;
  const dim3 grid((unsigned)((a->n_blocks + 127) / 128));
  const uint8_t *src = (const uint8_t *)a->src_mem;
  uint8_t *dst = (uint8_t *)a->dst_mem;
  const int64_t n = (int64_t)a->n_blocks;
#define ARGUS_REQUANT(O, N) hipLaunchKernelGGL((kivi_requant_kernel<O, N>), grid, dim3(128), 0, stream, src, dst, n)
  switch (a->old_bits * 16 + a->new_bits) {
    case 2 * 16 + 2: ARGUS_REQUANT(2, 2); break;
    case 2 * 16 + 4: ARGUS_REQUANT(2, 4); break;
    case 2 * 16 + 8: ARGUS_REQUANT(2, 8); break;
    case 4 * 16 + 2: ARGUS_REQUANT(4, 2); break;
    case 4 * 16 + 4: ARGUS_REQUANT(4, 4); break;
    case 4 * 16 + 8: ARGUS_REQUANT(4, 8); break;
    case 8 * 16 + 2: ARGUS_REQUANT(8, 2); break;
    case 8 * 16 + 4: ARGUS_REQUANT(8, 4); break;
    default: ARGUS_REQUANT(8, 8); break;
  }
#undef ARGUS_REQUANT
  ARGUS_HIP_CHECK(ctx, hipGetLastError());
  return ARGUS_HIP_OK;
}
