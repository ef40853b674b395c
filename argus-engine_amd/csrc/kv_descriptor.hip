// Descriptor-driven block formats on the device: the generic floor of `--kv-format`.
//
// Stand in for decode_via_descriptor / unpack_block_via_descriptor
// (engine/src/format/dtype_layout.rs:102-166, 285-300) and encode_via_descriptor with its two
// canonical encoders (302-396): block = [f16 scale][f16 min?][packed quants], vocabulary
// KVLayoutDesc { block_elems, bits, scale_layout, packing } (argus-extension-api lib.rs:1111-1159).
// Results are bit-identical to the CPU functions: products of a small integer and an f16 scale are
// exact in f32, the encoders use the same correctly rounded divide / reciprocal / round-half-away.
// Blocks are only 2-byte aligned (12 / 18 / 20 / 34 bytes), so they are read and written as 16-bit
// units.  32-element blocks (every named format) take four threads per block, eight elements each:
// a thread then stores or loads 16 or 32 contiguous bytes of the row and the wave's accesses are
// dense (one thread per block wrote 2-byte elements 64 bytes apart: 0.5 TB/s).  Other block sizes
// keep the one-thread-per-block kernels.
#include "argus_hip_internal.hpp"

namespace {

enum { kScaleNone = 0, kScaleF16 = 1, kScaleF16Min = 2 };
enum { kDense = 0, kNibble = 1, kByte = 2, kQuad = 3 };
constexpr int kMaxBlockElems = 64;

struct DescParams {
  int32_t block_elems, bits, scale_layout, packing, block_bytes;
  int64_t n_blocks;
};

__device__ __forceinline__ float half_bits_to_float(uint16_t b) { return (float)__builtin_bit_cast(_Float16, b); }

// The value is an f32 (as in the CPU functions) rounded once to the output type.  The empty asm
// keeps the compiler from evaluating int * half products in f16, which drops the sign of a zero
// product (0 * negative scale is -0.0).
template <typename OUT_T>
__device__ __forceinline__ OUT_T store_cast(float r) {
  asm("" : "+v"(r));
  return (OUT_T)r;
}

template <typename OUT_T>
__global__ __launch_bounds__(256) void desc_decode_kernel(const DescParams p, const uint16_t *src, OUT_T *dst) {
  const int64_t bi = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (bi >= p.n_blocks) return;
  const uint16_t *blk = src + bi * (p.block_bytes / 2);
  const int n = p.block_elems;
  const float scale = half_bits_to_float(blk[0]);
  const float mn = p.scale_layout == kScaleF16Min ? half_bits_to_float(blk[1]) : 0.0f;
  const uint16_t *qw = blk + (p.scale_layout == kScaleF16Min ? 2 : 1);  // packed quants, 16 bits at a time
  OUT_T *out = dst + bi * n;
  auto byte_at = [&](int i) -> uint32_t { return (qw[i >> 1] >> (8 * (i & 1))) & 0xffu; };
  if (p.packing == kNibble) {
    const int half = n / 2, zp = 1 << (p.bits - 1);
    const bool is_signed = p.scale_layout == kScaleF16;
    for (int i = 0; i < half; ++i) {
      const int b = (int)byte_at(i), lo = b & 0x0f, hi = b >> 4;
      if (is_signed) {
        out[i] = store_cast<OUT_T>(__fmul_rn((float)(lo - zp), scale));
        out[i + half] = store_cast<OUT_T>(__fmul_rn((float)(hi - zp), scale));
      } else {
        out[i] = store_cast<OUT_T>(__fadd_rn(__fmul_rn((float)lo, scale), mn));
        out[i + half] = store_cast<OUT_T>(__fadd_rn(__fmul_rn((float)hi, scale), mn));
      }
    }
  } else if (p.packing == kByte) {
    for (int i = 0; i < n; ++i) out[i] = store_cast<OUT_T>(__fmul_rn((float)(int)(int8_t)byte_at(i), scale));
  } else {
    for (int i = 0; i < n / 4; ++i) {
      const uint32_t b = byte_at(i);
      for (int j = 0; j < 4; ++j) out[i * 4 + j] = store_cast<OUT_T>(__fadd_rn(__fmul_rn((float)((b >> (2 * j)) & 3u), scale), mn));
    }
  }
}

typedef uint32_t u32_a2 __attribute__((aligned(2)));  // dword reads at 2-byte boundaries

// 32-element blocks, four threads per block: thread q decodes elements 8q .. 8q+7.
template <typename OUT_T>
__global__ __launch_bounds__(256) void desc_decode32_kernel(const DescParams p, const uint16_t *src, OUT_T *dst) {
  const int64_t gid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t bi = gid >> 2;
  const int q = (int)(gid & 3);
  if (bi >= p.n_blocks) return;
  const uint16_t *blk = src + bi * (p.block_bytes / 2);
  const float scale = half_bits_to_float(blk[0]);
  const bool has_min = p.scale_layout == kScaleF16Min;
  const float mn = has_min ? half_bits_to_float(blk[1]) : 0.0f;
  const uint16_t *qw = blk + (has_min ? 2 : 1);
  float r[8];
  if (p.packing == kNibble) {
    // element i < 16: low nibble of byte i; element 16 + i: high nibble of byte i
    const int zp = 1 << (p.bits - 1), sh = (q >> 1) * 4;
    const u32_a2 *cw = (const u32_a2 *)(qw + 4 * (q & 1));  // the thread's 8 code bytes as two dwords
#pragma unroll
    for (int k = 0; k < 2; ++k) {
      const uint32_t w = cw[k];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int code = (int)((w >> (8 * e + sh)) & 0x0fu);
        r[4 * k + e] = has_min ? __fadd_rn(__fmul_rn((float)code, scale), mn) : __fmul_rn((float)(code - zp), scale);
      }
    }
  } else if (p.packing == kByte) {
    const u32_a2 *cw = (const u32_a2 *)(qw + 4 * q);
#pragma unroll
    for (int k = 0; k < 2; ++k) {
      const uint32_t w = cw[k];
#pragma unroll
      for (int e = 0; e < 4; ++e) r[4 * k + e] = __fmul_rn((float)(int)(int8_t)((w >> (8 * e)) & 0xffu), scale);
    }
  } else {
    const uint32_t w = qw[q];  // bytes 2q, 2q+1: elements 8q .. 8q+7, two bits each
#pragma unroll
    for (int e = 0; e < 8; ++e) r[e] = __fadd_rn(__fmul_rn((float)((w >> (2 * e)) & 3u), scale), mn);
  }
  typedef OUT_T out8_t __attribute__((ext_vector_type(8)));
  out8_t o;
#pragma unroll
  for (int e = 0; e < 8; ++e) o[e] = store_cast<OUT_T>(r[e]);
  // written once and read by a later kernel: with the default policy this kernel ran at 0.61 of HBM
  // peak, with the write-once hint at 0.83-0.86
  __builtin_nontemporal_store(o, (out8_t *)(dst + bi * 32 + 8 * q));
}

__device__ __forceinline__ uint16_t float_to_half_bits(float x) { return __builtin_bit_cast(uint16_t, (_Float16)x); }

__global__ __launch_bounds__(256) void desc_encode_kernel(const DescParams p, const float *src, uint16_t *dst) {
  const int64_t bi = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (bi >= p.n_blocks) return;
  const int n = p.block_elems;
  float s[kMaxBlockElems];
  for (int i = 0; i < n; ++i) s[i] = src[bi * n + i];
  uint16_t *blk = dst + bi * (p.block_bytes / 2);
  if (p.packing == kNibble) {
    // encode_block_perblockf16_nibble (dtype_layout.rs:347-364)
    const float qmax = (float)((1 << (p.bits - 1)) - 1), qmin = -(float)(1 << (p.bits - 1));
    const int zp = 1 << (p.bits - 1), half = n / 2;
    float max_abs = 0.0f;
    for (int i = 0; i < n; ++i) max_abs = fmaxf(max_abs, fabsf(s[i]));
    const float d = __fdiv_rn(max_abs, qmax);
    const float id = d == 0.0f ? 0.0f : __fdiv_rn(1.0f, d);
    blk[0] = float_to_half_bits(d);
    for (int i = 0; i < half; i += 2) {
      uint32_t w = 0;
      for (int e = 0; e < 2; ++e) {
        const int v0 = (int)fminf(fmaxf(roundf(__fmul_rn(s[i + e], id)), qmin), qmax);
        const int v1 = (int)fminf(fmaxf(roundf(__fmul_rn(s[i + e + half], id)), qmin), qmax);
        w |= (uint32_t)(((v0 + zp) & 0xff) | (((v1 + zp) << 4) & 0xff)) << (8 * e);
      }
      blk[1 + i / 2] = (uint16_t)w;
    }
  } else {
    // encode_block_perblockf16withmin_quad (dtype_layout.rs:372-396)
    const float qmax = (float)((1u << p.bits) - 1u);
    const int per_byte = 8 / p.bits;
    float mn = __builtin_huge_valf(), mx = -__builtin_huge_valf();
    for (int i = 0; i < n; ++i) {
      mn = fminf(mn, s[i]);
      mx = fmaxf(mx, s[i]);
    }
    const float d = __fdiv_rn(__fsub_rn(mx, mn), qmax);
    const float id = d == 0.0f ? 0.0f : __fdiv_rn(1.0f, d);
    blk[0] = float_to_half_bits(d);
    blk[1] = float_to_half_bits(mn);
    for (int i = 0; i < n / per_byte; i += 2) {
      uint32_t w = 0;
      for (int e = 0; e < 2; ++e) {
        uint32_t byte = 0;
        for (int j = 0; j < per_byte; ++j) {
          const uint32_t qv = (uint32_t)fminf(fmaxf(roundf(__fmul_rn(__fsub_rn(s[(i + e) * per_byte + j], mn), id)), 0.0f), qmax);
          byte |= qv << (j * p.bits);
        }
        w |= (byte & 0xffu) << (8 * e);
      }
      blk[2 + i / 2] = (uint16_t)w;
    }
  }
}

// 32-element blocks, four threads per block: thread q quantises elements 8q .. 8q+7; the block's
// extrema and, for nibble packing, the partner's codes (byte i = element i | element 16 + i << 4)
// travel between the four lanes by shuffles.
__global__ __launch_bounds__(256) void desc_encode32_kernel(const DescParams p, const float *src, uint16_t *dst) {
  const int64_t gid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t bi = gid >> 2;
  const int q = (int)(gid & 3);
  if (bi >= p.n_blocks) return;  // the four lanes of a block leave together
  float s[8];
  {
    const float4_t a = *(const float4_t *)(src + bi * 32 + 8 * q), b = *(const float4_t *)(src + bi * 32 + 8 * q + 4);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      s[e] = a[e];
      s[4 + e] = b[e];
    }
  }
  uint16_t *blk = dst + bi * (p.block_bytes / 2);
  if (p.packing == kNibble) {
    const float qmax = (float)((1 << (p.bits - 1)) - 1), qmin = -(float)(1 << (p.bits - 1));
    const int zp = 1 << (p.bits - 1);
    float max_abs = 0.0f;
#pragma unroll
    for (int e = 0; e < 8; ++e) max_abs = fmaxf(max_abs, fabsf(s[e]));
    max_abs = fmaxf(max_abs, __shfl_xor(max_abs, 1, 64));
    max_abs = fmaxf(max_abs, __shfl_xor(max_abs, 2, 64));
    const float d = __fdiv_rn(max_abs, qmax);
    const float id = d == 0.0f ? 0.0f : __fdiv_rn(1.0f, d);
    uint32_t mine = 0;  // eight 4-bit codes
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int v = (int)fminf(fmaxf(roundf(__fmul_rn(s[e], id)), qmin), qmax);
      mine |= (uint32_t)((v + zp) & 0x0f) << (4 * e);
    }
    const uint32_t theirs = (uint32_t)__shfl_xor((int)mine, 2, 64);  // lanes 0, 1 receive elements 16 + ...
    if (q < 2) {
      if (q == 0) blk[0] = float_to_half_bits(d);
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const uint32_t b0 = ((mine >> (8 * k)) & 0x0fu) | (((theirs >> (8 * k)) & 0x0fu) << 4);
        const uint32_t b1 = ((mine >> (8 * k + 4)) & 0x0fu) | (((theirs >> (8 * k + 4)) & 0x0fu) << 4);
        blk[1 + 4 * q + k] = (uint16_t)(b0 | (b1 << 8));
      }
    }
  } else {
    const float qmax = 3.0f;  // quad packing is 2-bit
    float mn = __builtin_huge_valf(), mx = -__builtin_huge_valf();
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      mn = fminf(mn, s[e]);
      mx = fmaxf(mx, s[e]);
    }
    mn = fminf(mn, __shfl_xor(mn, 1, 64));
    mx = fmaxf(mx, __shfl_xor(mx, 1, 64));
    mn = fminf(mn, __shfl_xor(mn, 2, 64));
    mx = fmaxf(mx, __shfl_xor(mx, 2, 64));
    const float d = __fdiv_rn(__fsub_rn(mx, mn), qmax);
    const float id = d == 0.0f ? 0.0f : __fdiv_rn(1.0f, d);
    uint32_t w = 0;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const uint32_t qv = (uint32_t)fminf(fmaxf(roundf(__fmul_rn(__fsub_rn(s[e], mn), id)), 0.0f), qmax);
      w |= qv << (2 * e);
    }
    if (q == 0) {
      blk[0] = float_to_half_bits(d);
      blk[1] = float_to_half_bits(mn);
    }
    blk[2 + q] = (uint16_t)w;
  }
}

int check_desc(argus_hip_ctx *ctx, const argus_hip_kv_layout_desc *d, DescParams &p, const char *what) {
  int q;
  switch (d->packing) {
    case kNibble: q = (int)d->block_elems / 2; break;
    case kByte: q = (int)d->block_elems; break;
    case kQuad: q = (int)d->block_elems / 4; break;
    default: return argus_fail(ctx, ARGUS_HIP_ERR_UNSUPPORTED, "%s: packing %u has no block form", what, d->packing);
  }
  if (d->scale_layout != kScaleF16 && d->scale_layout != kScaleF16Min)
    return argus_fail(ctx, ARGUS_HIP_ERR_UNSUPPORTED, "%s: scale layout %u", what, d->scale_layout);
  const bool bits_ok = (d->packing == kNibble && d->bits >= 2 && d->bits <= 4) || (d->packing == kByte && d->bits == 8) ||
                       (d->packing == kQuad && d->bits == 2);
  if (!bits_ok || d->block_elems == 0 || d->block_elems > kMaxBlockElems || d->block_elems % 8)
    return argus_fail(ctx, ARGUS_HIP_ERR_UNSUPPORTED, "%s: block_elems %u bits %u", what, d->block_elems, (unsigned)d->bits);
  if (d->packing == kQuad && d->scale_layout != kScaleF16Min)
    return argus_fail(ctx, ARGUS_HIP_ERR_UNSUPPORTED, "%s: quad packing is min-bearing", what);
  p.block_elems = (int32_t)d->block_elems;
  p.bits = d->bits;
  p.scale_layout = (int32_t)d->scale_layout;
  p.packing = (int32_t)d->packing;
  p.block_bytes = q + (d->scale_layout == kScaleF16 ? 2 : 4);
  return ARGUS_HIP_OK;
}

}  // namespace

ARGUS_API int argus_hip_kv_decode_descriptor(argus_hip_ctx *ctx, void *stream, const argus_hip_kv_layout_desc *desc, const void *src,
                                             void *dst, int32_t dst_dtype, int64_t n_elems) {
  if (!ctx || !desc) return ARGUS_HIP_ERR_INVALID;
  DescParams p{};
  int rc = check_desc(ctx, desc, p, "kv_decode_descriptor");
  if (rc != ARGUS_HIP_OK) return rc;
  if (n_elems < 0 || n_elems % p.block_elems) return argus_fail(ctx, ARGUS_HIP_ERR_INVALID, "kv_decode_descriptor: %lld elements", (long long)n_elems);
  if (dst_dtype != ARGUS_HIP_F16 && dst_dtype != ARGUS_HIP_F32)
    return argus_fail(ctx, ARGUS_HIP_ERR_UNSUPPORTED, "kv_decode_descriptor: output dtype %d", dst_dtype);
  if (n_elems == 0) return ARGUS_HIP_OK;
  if (!src || !dst || ((uintptr_t)src & 1)) return argus_fail(ctx, ARGUS_HIP_ERR_INVALID, "kv_decode_descriptor: null or odd buffer");
  p.n_blocks = n_elems / p.block_elems;
  const bool fast = p.block_elems == 32 && ((uintptr_t)dst & 15) == 0 && p.n_blocks < (1ll << 37);
  const dim3 grid((unsigned)(((fast ? 4 : 1) * p.n_blocks + 255) / 256));
  if (dst_dtype == ARGUS_HIP_F16) {
    if (fast) hipLaunchKernelGGL(desc_decode32_kernel<_Float16>, grid, dim3(256), 0, (hipStream_t)stream, p, (const uint16_t *)src, (_Float16 *)dst);
    else hipLaunchKernelGGL(desc_decode_kernel<_Float16>, grid, dim3(256), 0, (hipStream_t)stream, p, (const uint16_t *)src, (_Float16 *)dst);
  } else {
    if (fast) hipLaunchKernelGGL(desc_decode32_kernel<float>, grid, dim3(256), 0, (hipStream_t)stream, p, (const uint16_t *)src, (float *)dst);
    else hipLaunchKernelGGL(desc_decode_kernel<float>, grid, dim3(256), 0, (hipStream_t)stream, p, (const uint16_t *)src, (float *)dst);
  }
  ARGUS_HIP_CHECK(ctx, hipGetLastError());
  return ARGUS_HIP_OK;
}

ARGUS_API int argus_hip_kv_encode_descriptor(argus_hip_ctx *ctx, void *stream, const argus_hip_kv_layout_desc *desc, const void *src,
                                             void *dst, int64_t n_elems) {
  if (!ctx || !desc) return ARGUS_HIP_ERR_INVALID;
  // the writable floor: q4_0-style (PerBlockF16 + Nibble) and q2_0-style (PerBlockF16WithMin + Quad)
  const bool nibble = desc->scale_layout == kScaleF16 && desc->packing == kNibble;
  const bool quad = desc->scale_layout == kScaleF16Min && desc->packing == kQuad;
  if (!nibble && !quad)
    return argus_fail(ctx, ARGUS_HIP_ERR_UNSUPPORTED, "kv_encode_descriptor: only PerBlockF16/Nibble or PerBlockF16WithMin/Quad, got %u/%u",
                      desc->scale_layout, desc->packing);
  DescParams p{};
  int rc = check_desc(ctx, desc, p, "kv_encode_descriptor");
  if (rc != ARGUS_HIP_OK) return rc;
  if (n_elems < 0 || n_elems % p.block_elems) return argus_fail(ctx, ARGUS_HIP_ERR_INVALID, "kv_encode_descriptor: %lld elements", (long long)n_elems);
  if (n_elems == 0) return ARGUS_HIP_OK;
  if (!src || !dst || ((uintptr_t)dst & 1) || ((uintptr_t)src & 3))
    return argus_fail(ctx, ARGUS_HIP_ERR_INVALID, "kv_encode_descriptor: null or misaligned buffer");
  p.n_blocks = n_elems / p.block_elems;
  if (p.block_elems == 32 && ((uintptr_t)src & 15) == 0 && p.n_blocks < (1ll << 37))
    hipLaunchKernelGGL(desc_encode32_kernel, dim3((unsigned)((4 * p.n_blocks + 255) / 256)), dim3(256), 0, (hipStream_t)stream, p,
                       (const float *)src, (uint16_t *)dst);
  else
    hipLaunchKernelGGL(desc_encode_kernel, dim3((unsigned)((p.n_blocks + 255) / 256)), dim3(256), 0, (hipStream_t)stream, p,
                       (const float *)src, (uint16_t *)dst);
  ARGUS_HIP_CHECK(ctx, hipGetLastError());
  return ARGUS_HIP_OK;
}
