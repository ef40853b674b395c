// The reference's dlopen plugin protocol for backend capabilities, so the engine can load this
// library as a capability plugin as it stands: `register_backend_caps_v2` returns, by value, the
// envelope BackendCapExportAbi { abi_version, count, vtables } whose entries
// BackendCapVTableAbi { name, category, vtable } point at one table per category
// (crates/argus-extension-api/src/lib.rs:1569-1578, 1726-1782; loader
// engine/src/capability/dynamic_backend_registry.rs:50-160).  Two entries: the fused dequant +
// attention capability (ATTENTION, QuantAttnVTable) and the KIVI container (CACHE, QuantCacheVTable,
// quant_cache.hip).  Host code only.
#include "argus_hip_internal.hpp"

#include <new>

namespace {

// Handle of the ATTENTION capability: a context of its own on the device that is current at `make`.
struct QuantAttnCap {
  argus_hip_ctx *ctx = nullptr;
};

}  // namespace

// The make arguments carry OpenCL handles in the reference (QuantAttnMakeArgs, lib.rs:1583-1592);
// nothing of them applies here and none is read.
ARGUS_API void *argus_hip_quant_attn_cap_make(const argus_hip_quant_attn_make_args *) {
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess) {
    (void)hipGetLastError();
    return nullptr;
  }
  QuantAttnCap *c = new (std::nothrow) QuantAttnCap();
  if (!c) return nullptr;
  if (argus_hip_create(device, &c->ctx) != ARGUS_HIP_OK) {
    delete c;
    return nullptr;
  }
  return c;
}
ARGUS_API void argus_hip_quant_attn_cap_drop(void *handle) {
  QuantAttnCap *c = (QuantAttnCap *)handle;
  if (!c) return;
  argus_hip_destroy(c->ctx);
  delete c;
}
ARGUS_API bool argus_hip_quant_attn_cap_has_kernel(void *handle, uint8_t bits) {
  const QuantAttnCap *c = (const QuantAttnCap *)handle;
  return c && argus_hip_has_quant_attn_kernel(c->ctx, bits) == 1;
}
// The CUDA twin answers true as well (crates/techniques/kivi/src/gpu_kivi_cuda.rs:44-46): the
// engine takes the kernel variant that needs no sub-group extension.
ARGUS_API bool argus_hip_quant_attn_cap_is_nosub_device(void *) { return true; }
ARGUS_API int32_t argus_hip_quant_attn_cap_attention_gen_quant(void *handle, const argus_hip_quant_attn_args *a) {
  const QuantAttnCap *c = (const QuantAttnCap *)handle;
  return c ? argus_hip_attention_gen_quant(c->ctx, a) : -1;
}
ARGUS_API int32_t argus_hip_quant_attn_cap_gather_update_quant(void *handle, const argus_hip_quant_gather_args *a) {
  const QuantAttnCap *c = (const QuantAttnCap *)handle;
  return c ? argus_hip_gather_update_quant(c->ctx, a) : -1;
}
ARGUS_API int32_t argus_hip_quant_attn_cap_dequant_flush(void *handle, const argus_hip_quant_dequant_flush_args *a) {
  const QuantAttnCap *c = (const QuantAttnCap *)handle;
  return c ? argus_hip_quant_dequant_flush(c->ctx, a) : -1;
}
ARGUS_API int32_t argus_hip_quant_attn_cap_scatter_residual(void *handle, const argus_hip_quant_scatter_residual_args *a) {
  const QuantAttnCap *c = (const QuantAttnCap *)handle;
  return c ? argus_hip_quant_scatter_residual(c->ctx, a) : -1;
}

ARGUS_API const argus_hip_quant_attn_vtable *argus_hip_quant_attn_get_vtable(void) {
  static const argus_hip_quant_attn_vtable vt = {argus_hip_quant_attn_cap_make,
                                                 argus_hip_quant_attn_cap_has_kernel,
                                                 argus_hip_quant_attn_cap_is_nosub_device,
                                                 argus_hip_quant_attn_cap_attention_gen_quant,
                                                 argus_hip_quant_attn_cap_gather_update_quant,
                                                 argus_hip_quant_attn_cap_dequant_flush,
                                                 argus_hip_quant_attn_cap_scatter_residual,
                                                 argus_hip_quant_attn_cap_drop};
  return &vt;
}

ARGUS_API argus_backend_cap_export_abi register_backend_caps_v2(void) {
  static const argus_backend_cap_vtable_abi entries[2] = {
      {ARGUS_HIP_CAP_NAME_ATTENTION, ARGUS_BACKEND_CAP_CATEGORY_ATTENTION, argus_hip_quant_attn_get_vtable()},
      {ARGUS_HIP_CAP_NAME_CACHE, ARGUS_BACKEND_CAP_CATEGORY_CACHE, argus_hip_quant_cache_get_vtable()},
  };
  return argus_backend_cap_export_abi{ARGUS_BACKEND_CAP_ABI_VERSION, 2, entries};
}
