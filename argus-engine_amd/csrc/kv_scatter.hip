// KV write path: F32 [seq_len, kv_heads, head_dim] rows -> HeadMajor cache rows.
//
// Stands in for Backend::kv_scatter_f32_to_f16 / _batch / _f32_batch
// (engine/src/backend.rs:425-545; device semantics engine/src/backend/cuda_pc/kernels.cu:305-360):
//   dst[h, write_pos_start + s, d] = cast(src[s, h, d]),  F16 cast is round-to-nearest-even.
// Each thread moves 4 consecutive elements of K and of V (16-byte loads, 8/16-byte stores).
#include "argus_hip_internal.hpp"

namespace {

template <bool TO_F16>
__global__ __launch_bounds__(256) void kv_scatter_kernel(
    const float *__restrict__ k_src, const float *__restrict__ v_src, void *__restrict__ k_dst,
    void *__restrict__ v_dst, int kv_heads, int head_dim, int64_t capacity, int write_pos_start,
    int seq_len) {
  const int vec_per_row = head_dim / 4;
  const int64_t total = (int64_t)seq_len * kv_heads * vec_per_row;
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const int c = (int)(i % vec_per_row) * 4;
  const int64_t row = i / vec_per_row;  // s * kv_heads + h
  const int h = (int)(row % kv_heads);
  const int64_t s = row / kv_heads;
  const int64_t so = row * head_dim + c;
  const int64_t dofs = ((int64_t)h * capacity + write_pos_start + s) * head_dim + c;
  const float4_t kv = *(const float4_t *)(k_src + so);
  const float4_t vv = *(const float4_t *)(v_src + so);
  if constexpr (TO_F16) {
    half4_t kh, vh;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      kh[e] = (_Float16)kv[e];
      vh[e] = (_Float16)vv[e];
    }
    *(half4_t *)((_Float16 *)k_dst + dofs) = kh;
    *(half4_t *)((_Float16 *)v_dst + dofs) = vh;
  } else {
    *(float4_t *)((float *)k_dst + dofs) = kv;
    *(float4_t *)((float *)v_dst + dofs) = vv;
  }
}

template <bool TO_F16>
int scatter(argus_hip_ctx *ctx, void *stream, const float *k_src, const float *v_src, void *k_dst,
            void *v_dst, int kv_heads, int head_dim, int capacity, int write_pos_start, int seq_len) {
  if (!ctx) return ARGUS_HIP_ERR_INVALID;
  if (!k_src || !v_src || !k_dst || !v_dst) return argus_fail(ctx, ARGUS_HIP_ERR_INVALID, "kv_scatter: null pointer");
  if (kv_heads <= 0 || head_dim <= 0 || head_dim % 4 || seq_len < 0 || write_pos_start < 0)
    return argus_fail(ctx, ARGUS_HIP_ERR_INVALID, "kv_scatter: kv_heads %d head_dim %d seq_len %d", kv_heads, head_dim, seq_len);
  if ((int64_t)write_pos_start + seq_len > capacity)
    return argus_fail(ctx, ARGUS_HIP_ERR_INVALID, "kv_scatter: write_pos %d + seq_len %d exceeds capacity %d",
                      write_pos_start, seq_len, capacity);
  if (seq_len == 0) return ARGUS_HIP_OK;
  const int64_t total = (int64_t)seq_len * kv_heads * (head_dim / 4);
  const int64_t blocks = (total + 255) / 256;
  if (blocks > 0x7fffffff) return argus_fail(ctx, ARGUS_HIP_ERR_UNSUPPORTED, "kv_scatter: too many rows");
  hipLaunchKernelGGL(kv_scatter_kernel<TO_F16>, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, k_src,
                     v_src, k_dst, v_dst, kv_heads, head_dim, (int64_t)capacity, write_pos_start, seq_len);
  ARGUS_HIP_CHECK(ctx, hipGetLastError());
  return ARGUS_HIP_OK;
}

}  // namespace

ARGUS_API int argus_hip_kv_scatter_f32_to_f16(argus_hip_ctx *ctx, void *stream, const float *k_src,
                                              const float *v_src, void *k_dst, void *v_dst, int32_t kv_heads,
                                              int32_t head_dim, int32_t capacity, int32_t write_pos) {
  return scatter<true>(ctx, stream, k_src, v_src, k_dst, v_dst, kv_heads, head_dim, capacity, write_pos, 1);
}

ARGUS_API int argus_hip_kv_scatter_f32_to_f16_batch(argus_hip_ctx *ctx, void *stream, const float *k_src,
                                                    const float *v_src, void *k_dst, void *v_dst,
                                                    int32_t kv_heads, int32_t head_dim, int32_t capacity,
                                                    int32_t write_pos_start, int32_t seq_len) {
  return scatter<true>(ctx, stream, k_src, v_src, k_dst, v_dst, kv_heads, head_dim, capacity, write_pos_start, seq_len);
}

ARGUS_API int argus_hip_kv_scatter_f32_batch(argus_hip_ctx *ctx, void *stream, const float *k_src,
                                             const float *v_src, float *k_dst, float *v_dst, int32_t kv_heads,
                                             int32_t head_dim, int32_t capacity, int32_t write_pos_start,
                                             int32_t seq_len) {
  return scatter<false>(ctx, stream, k_src, v_src, k_dst, v_dst, kv_heads, head_dim, capacity, write_pos_start, seq_len);
}
