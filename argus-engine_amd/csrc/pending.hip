// Entry points whose kernels are not built yet: they decline instead of computing.
#include "argus_hip_internal.hpp"

ARGUS_API int argus_hip_flash_attention_prefill(argus_hip_ctx *ctx, const argus_hip_prefill_args *) {
  return ctx ? 0 : ARGUS_HIP_ERR_INVALID;  // 0 = declined, caller runs its CPU path
}
ARGUS_API int argus_hip_has_quant_attn_kernel(const argus_hip_ctx *, uint8_t) { return 0; }
ARGUS_API int argus_hip_attention_gen_quant(argus_hip_ctx *ctx, const argus_hip_quant_attn_args *) {
  return argus_fail(ctx, ARGUS_HIP_ERR_UNSUPPORTED, "attention_gen_quant: not built");
}
ARGUS_API int argus_hip_attention_gen_quant_ex(argus_hip_ctx *ctx, const argus_hip_quant_attn_args *,
                                               const argus_hip_quant_attn_ext *) {
  return argus_fail(ctx, ARGUS_HIP_ERR_UNSUPPORTED, "attention_gen_quant_ex: not built");
}
ARGUS_API int argus_hip_gather_update_quant(argus_hip_ctx *ctx, const argus_hip_quant_gather_args *) {
  return argus_fail(ctx, ARGUS_HIP_ERR_UNSUPPORTED, "gather_update_quant: not built");
}
ARGUS_API int argus_hip_quant_flush(argus_hip_ctx *ctx, const argus_hip_quant_flush_args *) {
  return argus_fail(ctx, ARGUS_HIP_ERR_UNSUPPORTED, "quant_flush: not built");
}
