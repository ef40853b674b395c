// KIVI data movement into the F16 attention view [max_seq, kv_heads, head_dim] (sequence major):
// dequantise flushed blocks (keys: per-channel blocks, values: per-token blocks) and scatter the
// F32 residual ring.
//
// Stand in for CudaQuantAttnBackend::{dequant_flush, scatter_residual}
// (crates/argus-extension-api/src/lib.rs:3045-3103), kernel semantics
// crates/techniques/kivi/src/kivi_q2.cu:18-116 (out = f16(code * d + m); the product of a code of
// at most 8 bits and an f16 scale is exact in f32, so fused and unfused evaluation agree bit for
// bit).  The reference has these for Q2 only; all three widths are served here.
#include "kivi_common.hpp"

namespace {

using argus_kivi::kUnit;

template <int BITS>
__device__ __forceinline__ uint32_t code_at(const uint8_t *qs, int i) {
  if constexpr (BITS == 8) return qs[i];
  else if constexpr (BITS == 4) return (qs[i >> 1] >> (4 * (i & 1))) & 0xfu;
  else return (qs[i >> 2] >> (2 * (i & 3))) & 0x3u;
}

// Keys: block (h, g, ch) holds 32 tokens of one channel.  One workgroup takes the D blocks of one
// (head, group) -- contiguous in the block stream -- through LDS and writes 32 token rows of D halfs,
// so that both the reads and the writes are contiguous (a thread per block would write 2-byte
// elements kv_heads * D * 2 bytes apart).
template <int BITS>
__global__ __launch_bounds__(256) void kivi_dequant_key_kernel(const uint8_t *blocks, _Float16 *attn, int kv_heads, int D,
                                                               int groups, int tok_base, int64_t block_start) {
  constexpr int BB = 4 + 32 * BITS / 8;
  extern __shared__ __attribute__((aligned(16))) uint8_t tile[];  // D * BB bytes
  const int h = blockIdx.x / groups, g = blockIdx.x % groups;
  const uint32_t *src = (const uint32_t *)(blocks + (block_start + (int64_t)blockIdx.x * D) * BB);
  for (int i = threadIdx.x; i < D * BB / 4; i += blockDim.x) ((uint32_t *)tile)[i] = src[i];
  __syncthreads();
  const int cpr = D / 8;  // 16-byte chunks per output row
  for (int idx = threadIdx.x; idx < kUnit * cpr; idx += blockDim.x) {
    const int t = idx / cpr, c0 = (idx % cpr) * 8;
    half8_t o;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const uint8_t *blk = tile + (c0 + e) * BB;
      const float d = (float)*(const _Float16 *)blk, m = (float)*(const _Float16 *)(blk + 2);
      o[e] = (_Float16)fmaf((float)code_at<BITS>(blk + 4, t), d, m);
    }
    *(half8_t *)(attn + ((int64_t)(tok_base + g * kUnit + t) * kv_heads + h) * D + c0) = o;
  }
}

// Values: block (h, t, b) holds 32 channels of one token: 64 contiguous output bytes per block.
template <int BITS>
__global__ __launch_bounds__(256) void kivi_dequant_value_kernel(const uint8_t *blocks, _Float16 *attn, int kv_heads, int D,
                                                                 int flush_tokens, int tok_base, int64_t block_start) {
  constexpr int BB = 4 + 32 * BITS / 8;
  const int bpt = D / kUnit;
  const int64_t bid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (bid >= (int64_t)kv_heads * flush_tokens * bpt) return;
  const int b = (int)(bid % bpt);
  const int64_t tmp = bid / bpt;
  const int t = (int)(tmp % flush_tokens), h = (int)(tmp / flush_tokens);
  uint32_t raw[BB / 4];
  const uint32_t *src = (const uint32_t *)(blocks + (block_start + bid) * BB);
#pragma unroll
  for (int i = 0; i < BB / 4; ++i) raw[i] = src[i];
  const float d = (float)__builtin_bit_cast(_Float16, (uint16_t)(raw[0] & 0xffffu));
  const float m = (float)__builtin_bit_cast(_Float16, (uint16_t)(raw[0] >> 16));
  _Float16 *dst = attn + ((int64_t)(tok_base + t) * kv_heads + h) * D + b * kUnit;
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    half8_t o;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int i = 8 * c + e;  // channel inside the block
      const int bit = i * BITS;
      const uint32_t code = (raw[1 + bit / 32] >> (bit % 32)) & ((1u << BITS) - 1u);
      o[e] = (_Float16)fmaf((float)code, d, m);
    }
    *(half8_t *)(dst + 8 * c) = o;
  }
}

// Residual ring [kv_heads, res_cap, D] F32 -> rows tok_base .. tok_base + res_pos of the F16 view.
__global__ __launch_bounds__(256) void kivi_scatter_residual_kernel(const float *residual, _Float16 *attn, int kv_heads, int res_cap,
                                                                    int D, int res_pos, int tok_base) {
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int cpr = D / 4;
  if (idx >= (int64_t)kv_heads * res_pos * cpr) return;
  const int c = (int)(idx % cpr);
  const int64_t tmp = idx / cpr;
  const int h = (int)(tmp % kv_heads), t = (int)(tmp / kv_heads);  // head fastest: output rows stay contiguous
  const float4_t v = *(const float4_t *)(residual + ((int64_t)h * res_cap + t) * D + 4 * c);
  const half4_t o = {(_Float16)v[0], (_Float16)v[1], (_Float16)v[2], (_Float16)v[3]};
  *(half4_t *)(attn + ((int64_t)(tok_base + t) * kv_heads + h) * D + 4 * c) = o;
}

}  // namespace

ARGUS_API int argus_hip_quant_dequant_flush(argus_hip_ctx *ctx, const argus_hip_quant_dequant_flush_args *a) {
  if (!ctx || !a) return ARGUS_HIP_ERR_INVALID;
  if (a->bits != 2 && a->bits != 4 && a->bits != 8)
    return argus_fail(ctx, ARGUS_HIP_ERR_UNSUPPORTED, "dequant_flush unsupported for bits=%d", (int)a->bits);
  if (!a->q_blocks_mem || !a->attn_mem) return argus_fail(ctx, ARGUS_HIP_ERR_INVALID, "dequant_flush: null buffer");
  if (a->kv_heads == 0 || a->head_dim == 0 || a->head_dim % kUnit || a->head_dim > 1024)
    return argus_fail(ctx, ARGUS_HIP_ERR_INVALID, "dequant_flush: kv_heads %zu head_dim %zu", a->kv_heads, a->head_dim);
  if ((a->q_blocks_mem & 3) || (a->attn_mem & 15))
    return argus_fail(ctx, ARGUS_HIP_ERR_INVALID, "dequant_flush: misaligned buffer");
  if (a->n_groups_or_tokens == 0) return ARGUS_HIP_OK;
  hipStream_t stream = (hipStream_t)a->stream;
  const uint8_t *blocks = (const uint8_t *)a->q_blocks_mem;
  _Float16 *attn = (_Float16 *)a->attn_mem;
  const int H = (int)a->kv_heads, D = (int)a->head_dim, n = (int)a->n_groups_or_tokens, tb = (int)a->tok_base;
  const int64_t bs = (int64_t)a->block_start;
  if (a->is_key) {
    const int64_t wgs = (int64_t)H * n;
    if (wgs > 0x7fffffff) return argus_fail(ctx, ARGUS_HIP_ERR_UNSUPPORTED, "dequant_flush: grid too large");
    const size_t lds = (size_t)D * (4 + 32 * a->bits / 8);
    switch (a->bits) {
      case 2: hipLaunchKernelGGL(kivi_dequant_key_kernel<2>, dim3((unsigned)wgs), dim3(256), lds, stream, blocks, attn, H, D, n, tb, bs); break;
      case 4: hipLaunchKernelGGL(kivi_dequant_key_kernel<4>, dim3((unsigned)wgs), dim3(256), lds, stream, blocks, attn, H, D, n, tb, bs); break;
      default: hipLaunchKernelGGL(kivi_dequant_key_kernel<8>, dim3((unsigned)wgs), dim3(256), lds, stream, blocks, attn, H, D, n, tb, bs); break;
    }
  } else {
    const int64_t nblk = (int64_t)H * n * (D / kUnit);
    const dim3 grid((unsigned)((nblk + 255) / 256));
    switch (a->bits) {
      case 2: hipLaunchKernelGGL(kivi_dequant_value_kernel<2>, grid, dim3(256), 0, stream, blocks, attn, H, D, n, tb, bs); break;
      case 4: hipLaunchKernelGGL(kivi_dequant_value_kernel<4>, grid, dim3(256), 0, stream, blocks, attn, H, D, n, tb, bs); break;
      default: hipLaunchKernelGGL(kivi_dequant_value_kernel<8>, grid, dim3(256), 0, stream, blocks, attn, H, D, n, tb, bs); break;
    }
  }
  ARGUS_HIP_CHECK(ctx, hipGetLastError());
  return ARGUS_HIP_OK;
}

ARGUS_API int argus_hip_quant_scatter_residual(argus_hip_ctx *ctx, const argus_hip_quant_scatter_residual_args *a) {
  if (!ctx || !a) return ARGUS_HIP_ERR_INVALID;
  if (!a->res_mem || !a->attn_mem) return argus_fail(ctx, ARGUS_HIP_ERR_INVALID, "scatter_residual: null buffer");
  if (a->kv_heads == 0 || a->head_dim == 0 || a->head_dim % 4 || a->res_pos > a->res_cap)
    return argus_fail(ctx, ARGUS_HIP_ERR_INVALID, "scatter_residual: head_dim %zu res_pos %zu res_cap %zu", a->head_dim, a->res_pos,
                      a->res_cap);
  if ((a->res_mem & 15) || (a->attn_mem & 7)) return argus_fail(ctx, ARGUS_HIP_ERR_INVALID, "scatter_residual: misaligned buffer");
  if (a->res_pos == 0) return ARGUS_HIP_OK;
  const int64_t total = (int64_t)a->kv_heads * a->res_pos * (a->head_dim / 4);
  hipLaunchKernelGGL(kivi_scatter_residual_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, (hipStream_t)a->stream,
                     (const float *)a->res_mem, (_Float16 *)a->attn_mem, (int)a->kv_heads, (int)a->res_cap, (int)a->head_dim,
                     (int)a->res_pos, (int)a->tok_base);
  ARGUS_HIP_CHECK(ctx, hipGetLastError());
  return ARGUS_HIP_OK;
}
