"""CPU-side checks of the C ABI: the library loads, exports every declared symbol, and
degrades to error codes (never a crash) without a device or with null arguments."""
import ctypes as C
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "argus_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(argus_hip_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    import argus_hip as A
    declared = _declared_symbols()
    assert len(declared) >= 20
    for name in declared:
        assert hasattr(A.lib, name), "missing export " + name
    assert sorted(A.EXPORTED_SYMBOLS) == declared
    assert A.lib.argus_hip_abi_version() == 2


def test_struct_layouts_match_header_field_order():
    # the ctypes mirrors must list the same fields in the same order as the header structs
    import argus_hip as A
    text = open(os.path.join(ROOT, "include", "argus_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    pairs = {"argus_hip_attention_gen_args": A.AttentionGenArgs, "argus_hip_prefill_args": A.PrefillArgs,
             "argus_hip_pfa_args": A.PfaArgs, "argus_hip_kv_layout_desc": A.KvLayoutDesc,
             "argus_hip_quant_attn_args": A.QuantAttnArgs, "argus_hip_quant_attn_ext": A.QuantAttnExt,
             "argus_hip_quant_gather_args": A.QuantGatherArgs, "argus_hip_quant_flush_args": A.QuantFlushArgs,
             "argus_hip_quant_dequant_flush_args": A.QuantDequantFlushArgs,
             "argus_hip_quant_scatter_residual_args": A.QuantScatterResidualArgs,
             "argus_hip_score_reduce_args": A.ScoreReduceArgs, "argus_hip_device_info": A.DeviceInfo,
             "argus_hip_create_opts": A.CreateOpts, "argus_hip_decode_plan": A.DecodePlan,
             "argus_hip_quant_requant_args": A.QuantRequantArgs, "argus_hip_quant_attn_make_args": A.QuantAttnMakeArgs,
             "argus_backend_cap_vtable_abi": A.BackendCapVTableAbi, "argus_backend_cap_export_abi": A.BackendCapExportAbi,
             "argus_hip_quant_cache_make_args": A.QuantCacheMakeArgs,
             "argus_hip_quant_cache_update_args": A.QuantCacheUpdateArgs,
             "argus_hip_quant_cache_view_out": A.QuantCacheViewOut,
             "argus_hip_quant_cache_raw_buffers_out": A.QuantCacheRawBuffersOut}
    for cname, cls in pairs.items():
        body = re.search(r"typedef struct %s \{(.*?)\} %s;" % (cname, cname), text, re.S).group(1)
        fields = []
        for decl in body.split(";"):
            decl = decl.strip()
            if not decl:
                continue
            for part in decl.split(","):
                fields.append(re.findall(r"([A-Za-z_][A-Za-z0-9_]*)\s*(?:\[\d+\])?\s*$", part.strip())[0])
        assert fields == [f[0] for f in cls._fields_], cname


def test_quant_cache_vtable_lists_the_exports_in_the_reference_order():
    # QuantCacheVTable, crates/argus-extension-api/src/lib.rs:2068-2090: make, current_pos, capacity,
    # current_bits, update, flush_if_full, assemble_view, get_raw_buffers, transition_bits, drop
    import argus_hip as A
    vt = A.lib.argus_hip_quant_cache_get_vtable().contents
    order = ["make", "current_pos", "capacity", "current_bits", "update", "flush_if_full", "assemble_view",
             "get_raw_buffers", "transition_bits", "drop"]
    assert [f[0] for f in A.QuantCacheVTable._fields_] == order
    for name in order:
        fn = getattr(A.lib, "argus_hip_quant_cache_" + name)
        assert getattr(vt, name) == C.cast(fn, C.c_void_p).value, name
    # a null handle never crashes
    null = C.c_void_p()
    assert A.lib.argus_hip_quant_cache_current_pos(null) == 0 and A.lib.argus_hip_quant_cache_capacity(null) == 0
    assert A.lib.argus_hip_quant_cache_update(null, None) < 0 and A.lib.argus_hip_quant_cache_flush_if_full(null) < 0
    assert A.lib.argus_hip_quant_cache_transition_bits(null, 4) < 0
    assert not A.lib.argus_hip_quant_cache_get_raw_buffers(null, None)
    assert not A.lib.argus_hip_quant_cache_make(None)
    A.lib.argus_hip_quant_cache_drop(null)


def test_plugin_envelope_follows_the_reference_dlopen_protocol():
    # register_backend_caps_v2 -> BackendCapExportAbi { abi_version 2, count, vtables } of
    # BackendCapVTableAbi { name, category, vtable } (crates/argus-extension-api/src/lib.rs:1569-1578,
    # 1752-1782; loader engine/src/capability/dynamic_backend_registry.rs:50-160: version check, non-null
    # vtables, known categories, unique names).
    import argus_hip as A
    env = A.lib.register_backend_caps_v2()
    assert env.abi_version == 2 and env.count == 2 and bool(env.vtables)
    entries = [env.vtables[i] for i in range(env.count)]
    assert [(e.name, e.category) for e in entries] == [(b"kivi_hip", 1), (b"kivi_cache_hip", 2)]
    assert entries[0].vtable == C.cast(A.lib.argus_hip_quant_attn_get_vtable(), C.c_void_p).value
    assert entries[1].vtable == C.cast(A.lib.argus_hip_quant_cache_get_vtable(), C.c_void_p).value
    # QuantAttnVTable order, lib.rs:1726-1746
    vt = A.lib.argus_hip_quant_attn_get_vtable().contents
    names = {"make": "make", "has_quant_attn_kernel": "has_kernel", "is_nosub_device": "is_nosub_device",
             "attention_gen_quant": "attention_gen_quant", "gather_update_quant": "gather_update_quant",
             "dequant_flush": "dequant_flush", "scatter_residual": "scatter_residual", "drop": "drop"}
    assert [f[0] for f in A.QuantAttnVTable._fields_] == list(names)
    for field, sym in names.items():
        assert getattr(vt, field) == C.cast(getattr(A.lib, "argus_hip_quant_attn_cap_" + sym), C.c_void_p).value, field
    # a degraded (null) handle answers -1 / false without crashing (engine/tests/gate_c_kivi_backend_cap.rs:90-146)
    null = C.c_void_p()
    assert not A.lib.argus_hip_quant_attn_cap_has_kernel(null, 2)
    assert A.lib.argus_hip_quant_attn_cap_attention_gen_quant(null, None) == -1
    assert A.lib.argus_hip_quant_attn_cap_gather_update_quant(null, None) == -1
    assert A.lib.argus_hip_quant_attn_cap_dequant_flush(null, None) == -1
    assert A.lib.argus_hip_quant_attn_cap_scatter_residual(null, None) == -1
    A.lib.argus_hip_quant_attn_cap_drop(null)


def test_degraded_without_device_or_context():
    # mirrors engine/tests/gate_c_kivi_backend_cap.rs:90-146: with no GPU every op returns a
    # negative code without crashing.
    import argus_hip as A
    import torch
    if torch.cuda.is_available():
        pytest.skip("a device is present; the no-device path is exercised on CPU-only hosts")
    h = C.c_void_p()
    assert A.lib.argus_hip_create(0, C.byref(h)) == A.ERR_RUNTIME and not h.value
    assert A.lib.argus_hip_attention_gen(None, None) == A.ERR_INVALID
    assert A.lib.argus_hip_score_reduce(None, None) == A.ERR_INVALID
    assert A.lib.argus_hip_attention_gen_quant(None, None) < 0
    assert A.lib.argus_hip_flash_attention_prefill(None, None) < 0
    assert A.lib.argus_hip_kv_scatter_f32_to_f16(None, None, None, None, None, None, 1, 64, 8, 0) == A.ERR_INVALID
    assert A.lib.argus_hip_destroy(None) == A.ERR_INVALID
    opts = A.CreateOpts(16, 32, 128, 32768)
    assert A.lib.argus_hip_create_ex(0, C.byref(opts), C.byref(h)) == A.ERR_RUNTIME and not h.value
    assert A.lib.argus_hip_buffer_shift(None, None, None, None, 16) == A.ERR_INVALID
    assert A.lib.argus_hip_write_buffer_range(None, None, None, 0, None, 16) == A.ERR_INVALID
    assert A.lib.argus_hip_reserve_workspace(None, 1 << 20) == A.ERR_INVALID
    assert A.lib.argus_hip_last_decode_plan(None, None) == A.ERR_INVALID
    with pytest.raises(A.ArgusHipError):
        A.Context(0)
