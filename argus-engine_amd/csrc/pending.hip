// Entry points whose kernels are not built yet: they decline instead of computing.
#include "argus_hip_internal.hpp"

ARGUS_API int argus_hip_flash_attention_prefill(argus_hip_ctx *ctx, const argus_hip_prefill_args *) {
  return ctx ? 0 : ARGUS_HIP_ERR_INVALID;  // 0 = declined, caller runs its CPU path
}
