// Launch parameters shared by the KIVI fused-decode kernels.
#pragma once

#include "decode_common.hpp"

namespace argus_kivi {

using argus_decode::DecodeParams;

constexpr int kUnit = 32;  // tokens per unit == codec group size (QKKV)

struct KiviParams {
  DecodeParams d;          // q/out/scores/ws/nsplit/scale/softcap/group/heads as for decode
  const uint8_t *qk;
  const uint8_t *qv;
  const void *res_k;
  const void *res_v;
  int32_t head_dim, q_tokens, res_tokens, res_cap;
  int32_t units_total, units_per_split;
  int32_t res_f16;
  int64_t qk_bs, qv_bs;  // bytes between consecutive sequences' block streams
  int64_t res_bs;        // elements between consecutive sequences' residual windows
};

// Matrix-core variant (kivi_mfma.hip): head_dim 64 / 128, up to 16 query heads per KV head,
// 16-byte aligned block streams.
bool kivi_mfma_supported(const KiviParams &kp);
int launch_kivi_mfma(argus_hip_ctx *ctx, KiviParams &kp, int bits, int batch, hipStream_t stream);

}  // namespace argus_kivi
