"""ctypes binding of libargus_hip.so (the C ABI declared in include/argus_hip.h).

This module is plumbing for tests and bench.py: it loads the in-tree shared library, mirrors
the argument structs field for field and passes raw device pointers (torch tensors are used
only as device memory and for the stream handle).  There is no fallback: if the library is
missing, importing this module raises.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
# ARGUS_HIP_LIB selects another build of the same library (profiling / A-B runs).
LIB_PATH = os.environ.get("ARGUS_HIP_LIB") or os.path.join(_HERE, "libargus_hip.so")

OK, ERR_INVALID, ERR_UNSUPPORTED, ERR_RUNTIME, ERR_NOMEM = 0, -1, -2, -3, -4
F32, F16 = 0, 1
Q4_0, Q4_1, Q8_0, Q2_0 = 2, 3, 4, 5  # block-quantised cache rows (attention_gen)
HEAD_MAJOR, SEQ_MAJOR = 0, 1
# KVLayoutDesc tuples (block_elems, bits, scale_layout, packing) of the named --kv-format formats,
# crates/argus-extension-api/src/lib.rs:1111-1159: scale_layout 1 PerBlockF16 / 2 PerBlockF16WithMin,
# packing 1 Nibble / 2 Byte / 3 Quad.
DESC_Q4_0 = (32, 4, 1, 1)
DESC_Q4_1 = (32, 4, 2, 1)
DESC_Q8_0 = (32, 8, 1, 2)
DESC_Q2_0 = (32, 2, 2, 3)

EXPORTED_SYMBOLS = [
    "argus_hip_create", "argus_hip_destroy", "argus_hip_abi_version", "argus_hip_last_error",
    "argus_hip_get_device_info", "argus_hip_kernel_timing_begin", "argus_hip_kernel_timing_end",
    "argus_hip_malloc", "argus_hip_free", "argus_hip_write_buffer",
    "argus_hip_read_buffer", "argus_hip_copy_slice", "argus_hip_synchronize",
    "argus_hip_create_ex", "argus_hip_reserve_workspace", "argus_hip_kernel_timing_end2",
    "argus_hip_write_buffer_range", "argus_hip_buffer_shift", "argus_hip_last_decode_plan",
    "argus_hip_attention_gen", "argus_hip_attention_gen_noalloc", "argus_hip_flash_attention_prefill", "argus_hip_prefill_attention_scores",
    "argus_hip_has_quant_attn_kernel", "argus_hip_attention_gen_quant",
    "argus_hip_attention_gen_quant_ex", "argus_hip_gather_update_quant", "argus_hip_quant_flush",
    "argus_hip_quant_dequant_flush", "argus_hip_quant_scatter_residual",
    "argus_hip_score_reduce", "argus_hip_score_reduce_per_layer",
    "argus_hip_score_reduce_ex", "argus_hip_score_reduce_per_layer_ex",
    "argus_hip_kv_scatter_f32_to_f16", "argus_hip_kv_scatter_f32_to_f16_batch",
    "argus_hip_kv_scatter_f32_batch", "argus_hip_kv_decode_descriptor", "argus_hip_kv_encode_descriptor",
    "argus_hip_attention_gen_desc", "argus_hip_quant_requant",
    "argus_hip_quant_cache_make", "argus_hip_quant_cache_drop", "argus_hip_quant_cache_current_pos",
    "argus_hip_quant_cache_capacity", "argus_hip_quant_cache_current_bits", "argus_hip_quant_cache_update",
    "argus_hip_quant_cache_flush_if_full", "argus_hip_quant_cache_assemble_view",
    "argus_hip_quant_cache_get_raw_buffers", "argus_hip_quant_cache_transition_bits",
    "argus_hip_quant_cache_get_vtable",
    "argus_hip_quant_attn_cap_make", "argus_hip_quant_attn_cap_drop", "argus_hip_quant_attn_cap_has_kernel",
    "argus_hip_quant_attn_cap_is_nosub_device", "argus_hip_quant_attn_cap_attention_gen_quant",
    "argus_hip_quant_attn_cap_gather_update_quant", "argus_hip_quant_attn_cap_dequant_flush",
    "argus_hip_quant_attn_cap_scatter_residual", "argus_hip_quant_attn_get_vtable",
]

if not os.path.exists(LIB_PATH):
    raise ImportError(
        "libargus_hip.so is not built: run `python -c 'import __graft_entry__ as g; g.build()'` "
        "(or `make -C argus-engine_amd/csrc`) first; there is no CPU fallback")

# torch bundles its own HIP runtime under the same soname as /opt/rocm's; whichever is loaded
# first serves the whole process.  Import torch first so the tensors handed to the library and
# the library's own launches go through one runtime.
import torch  # noqa: E402,F401

lib = C.CDLL(LIB_PATH)


class DeviceInfo(C.Structure):
    _fields_ = [("compute_units", C.c_int32), ("clock_mhz", C.c_int32),
                ("wavefront_size", C.c_int32), ("lds_bytes_per_block", C.c_int32),
                ("hbm_bytes", C.c_int64), ("name", C.c_char * 128), ("gcn_arch", C.c_char * 64)]


class CreateOpts(C.Structure):
    _fields_ = [("max_batch", C.c_int32), ("max_heads_q", C.c_int32), ("max_head_dim", C.c_int32),
                ("max_seq_len", C.c_int32)]


class DecodePlan(C.Structure):
    _fields_ = [("nsplit", C.c_int32), ("chunk", C.c_int32), ("wgs_per_cu", C.c_int32),
                ("lds_bytes", C.c_int32), ("launches", C.c_int32), ("kernel", C.c_int32),
                ("staged_scores", C.c_int32)]


class AttentionGenArgs(C.Structure):
    _fields_ = [("stream", C.c_void_p), ("q", C.c_void_p), ("k_cache", C.c_void_p),
                ("v_cache", C.c_void_p), ("out", C.c_void_p), ("scores_out", C.c_void_p),
                ("kv_index", C.c_void_p),
                ("num_heads_q", C.c_int32), ("num_heads_kv", C.c_int32), ("head_dim", C.c_int32),
                ("cache_seq_len", C.c_int32), ("capacity", C.c_int32), ("kv_start", C.c_int32),
                ("layout", C.c_int32), ("kv_dtype", C.c_int32), ("batch", C.c_int32),
                ("score_stride", C.c_int32),
                ("q_batch_stride", C.c_int64), ("out_batch_stride", C.c_int64),
                ("kv_batch_stride", C.c_int64), ("score_batch_stride", C.c_int64),
                ("index_batch_stride", C.c_int64),
                ("softcap", C.c_float), ("scale", C.c_float),
                ("score_stats", C.c_void_p), ("stats_batch_stride", C.c_int64)]


class PrefillArgs(C.Structure):
    _fields_ = [("stream", C.c_void_p), ("q", C.c_void_p), ("k_cache", C.c_void_p),
                ("v_cache", C.c_void_p), ("out", C.c_void_p),
                ("n_heads_q", C.c_int32), ("n_heads_kv", C.c_int32), ("seq_len", C.c_int32),
                ("cache_seq_len", C.c_int32), ("head_dim", C.c_int32), ("kv_capacity", C.c_int32),
                ("batch_size", C.c_int32), ("is_head_major", C.c_int32), ("q_dtype", C.c_int32),
                ("kv_dtype", C.c_int32), ("out_dtype", C.c_int32), ("window", C.c_int32)]


class PfaArgs(C.Structure):
    _fields_ = [("stream", C.c_void_p), ("q", C.c_void_p), ("k", C.c_void_p), ("k_dtype", C.c_int32),
                ("n_heads_q", C.c_int32), ("n_heads_kv", C.c_int32), ("head_dim", C.c_int32),
                ("seq_len", C.c_int32), ("cache_seq_len", C.c_int32), ("k_pos_stride", C.c_int64),
                ("kv_head_stride", C.c_int64), ("q_start_pos", C.c_int32), ("q_window", C.c_int32),
                ("has_window", C.c_int32), ("window", C.c_int32), ("sum_out", C.c_void_p),
                ("per_row_out", C.c_void_p), ("per_row_per_head", C.c_int32)]


class QuantAttnArgs(C.Structure):
    _fields_ = [("stream", C.c_void_p), ("q_mem", C.c_uint64), ("qk_mem", C.c_uint64),
                ("qv_mem", C.c_uint64), ("res_k_mem", C.c_uint64), ("res_v_mem", C.c_uint64),
                ("out_mem", C.c_uint64), ("scores_out", C.c_void_p), ("scores_len", C.c_size_t),
                ("num_heads_q", C.c_size_t), ("num_heads_kv", C.c_size_t), ("head_dim", C.c_size_t),
                ("q_tokens", C.c_size_t), ("res_tokens", C.c_size_t), ("res_cap", C.c_size_t),
                ("scale", C.c_float), ("bits", C.c_uint8)]


class QuantAttnExt(C.Structure):
    _fields_ = [("scores_dev", C.c_uint64), ("score_stride", C.c_size_t),
                ("res_dtype", C.c_int32), ("softcap", C.c_float), ("batch", C.c_int32),
                ("block_batch_stride_bytes", C.c_int64), ("res_batch_stride", C.c_int64),
                ("score_batch_stride", C.c_int64), ("score_stats_dev", C.c_uint64)]


class ScoreReduceExt(C.Structure):
    _fields_ = [("stats", C.c_uint64)]


class QuantGatherArgs(C.Structure):
    _fields_ = [("stream", C.c_void_p), ("input_mem", C.c_uint64), ("residual_mem", C.c_uint64),
                ("kv_heads", C.c_size_t), ("res_cap", C.c_size_t), ("head_dim", C.c_size_t),
                ("seq_len", C.c_size_t), ("res_pos", C.c_size_t)]


class QuantFlushArgs(C.Structure):
    _fields_ = [("stream", C.c_void_p), ("res_k_mem", C.c_uint64), ("res_v_mem", C.c_uint64),
                ("qk_mem", C.c_uint64), ("qv_mem", C.c_uint64), ("kv_heads", C.c_size_t),
                ("res_cap", C.c_size_t), ("head_dim", C.c_size_t), ("flush_tokens", C.c_size_t),
                ("k_block_start", C.c_size_t), ("v_block_start", C.c_size_t), ("bits", C.c_uint8),
                ("out_res_cap", C.c_size_t)]


class QuantDequantFlushArgs(C.Structure):
    _fields_ = [("stream", C.c_void_p), ("q_blocks_mem", C.c_uint64), ("attn_mem", C.c_uint64),
                ("kv_heads", C.c_size_t), ("head_dim", C.c_size_t), ("n_groups_or_tokens", C.c_size_t),
                ("tok_base", C.c_size_t), ("block_start", C.c_size_t), ("bits", C.c_uint8),
                ("is_key", C.c_uint8)]


class QuantRequantArgs(C.Structure):
    _fields_ = [("stream", C.c_void_p), ("src_mem", C.c_uint64), ("dst_mem", C.c_uint64),
                ("n_blocks", C.c_size_t), ("old_bits", C.c_uint8), ("new_bits", C.c_uint8)]


class QuantCacheMakeArgs(C.Structure):
    _fields_ = [("ctx", C.c_void_p), ("device", C.c_void_p), ("stream", C.c_void_p), ("build_opts", C.c_char_p),
                ("kv_heads", C.c_size_t), ("head_dim", C.c_size_t), ("max_seq_len", C.c_size_t),
                ("residual_size", C.c_size_t), ("bits", C.c_uint8)]


class QuantCacheUpdateArgs(C.Structure):
    _fields_ = [("stream", C.c_void_p), ("k_in_mem", C.c_void_p), ("v_in_mem", C.c_void_p), ("seq_len", C.c_size_t)]


class QuantCacheViewOut(C.Structure):
    _fields_ = [("k_mem", C.c_void_p), ("v_mem", C.c_void_p), ("tokens", C.c_size_t), ("layout", C.c_uint32)]


class QuantCacheRawBuffersOut(C.Structure):
    _fields_ = [("qk_mem", C.c_void_p), ("qv_mem", C.c_void_p), ("res_k_mem", C.c_void_p), ("res_v_mem", C.c_void_p),
                ("q_tokens", C.c_size_t), ("res_tokens", C.c_size_t), ("res_cap", C.c_size_t), ("bits", C.c_uint8)]


class QuantCacheVTable(C.Structure):
    _fields_ = [(n, C.c_void_p) for n in ("make", "current_pos", "capacity", "current_bits", "update", "flush_if_full",
                                          "assemble_view", "get_raw_buffers", "transition_bits", "drop")]


class QuantAttnMakeArgs(C.Structure):
    _fields_ = [("cl_ctx", C.c_void_p), ("device", C.c_void_p), ("build_opts", C.c_char_p)]


class QuantAttnVTable(C.Structure):
    _fields_ = [(n, C.c_void_p) for n in ("make", "has_quant_attn_kernel", "is_nosub_device", "attention_gen_quant",
                                          "gather_update_quant", "dequant_flush", "scatter_residual", "drop")]


class BackendCapVTableAbi(C.Structure):
    _fields_ = [("name", C.c_char_p), ("category", C.c_uint32), ("vtable", C.c_void_p)]


class BackendCapExportAbi(C.Structure):
    _fields_ = [("abi_version", C.c_uint32), ("count", C.c_size_t), ("vtables", C.POINTER(BackendCapVTableAbi))]


class QuantScatterResidualArgs(C.Structure):
    _fields_ = [("stream", C.c_void_p), ("res_mem", C.c_uint64), ("attn_mem", C.c_uint64),
                ("kv_heads", C.c_size_t), ("res_cap", C.c_size_t), ("head_dim", C.c_size_t),
                ("res_pos", C.c_size_t), ("tok_base", C.c_size_t)]


class KvLayoutDesc(C.Structure):
    _fields_ = [("block_elems", C.c_uint32), ("bits", C.c_uint8), ("scale_layout", C.c_uint32),
                ("packing", C.c_uint32)]


class ScoreReduceArgs(C.Structure):
    _fields_ = [("stream", C.c_void_p), ("score_buf", C.c_uint64), ("importance", C.c_uint64),
                ("head_importance", C.c_uint64), ("decay_factor", C.c_float),
                ("n_layers", C.c_size_t), ("n_heads_q", C.c_size_t), ("n_kv_heads", C.c_size_t),
                ("cache_seq_len", C.c_size_t), ("score_stride", C.c_size_t),
                ("max_seq_len", C.c_size_t), ("layer_flat_importance", C.c_uint64)]


def _bind():
    vp, i32 = C.c_void_p, C.c_int32
    lib.argus_hip_create.argtypes = [C.c_int, C.POINTER(vp)]
    lib.argus_hip_create_ex.argtypes = [C.c_int, C.POINTER(CreateOpts), C.POINTER(vp)]
    lib.argus_hip_reserve_workspace.argtypes = [vp, C.c_size_t]
    lib.argus_hip_kernel_timing_end2.argtypes = [vp, C.POINTER(C.c_float), C.POINTER(C.c_float), i32, C.POINTER(i32)]
    lib.argus_hip_write_buffer_range.argtypes = [vp, vp, vp, C.c_size_t, vp, C.c_size_t]
    lib.argus_hip_buffer_shift.argtypes = [vp, vp, vp, vp, C.c_size_t]
    lib.argus_hip_last_decode_plan.argtypes = [vp, C.POINTER(DecodePlan)]
    lib.argus_hip_destroy.argtypes = [vp]
    lib.argus_hip_abi_version.argtypes = []
    lib.argus_hip_last_error.argtypes = [vp]
    lib.argus_hip_last_error.restype = C.c_char_p
    lib.argus_hip_get_device_info.argtypes = [vp, C.POINTER(DeviceInfo)]
    lib.argus_hip_kernel_timing_begin.argtypes = [vp, i32]
    lib.argus_hip_kernel_timing_end.argtypes = [vp, C.POINTER(C.c_float), i32, C.POINTER(i32)]
    lib.argus_hip_malloc.argtypes = [vp, C.c_size_t, C.POINTER(vp)]
    lib.argus_hip_free.argtypes = [vp, vp]
    lib.argus_hip_write_buffer.argtypes = [vp, vp, vp, vp, C.c_size_t]
    lib.argus_hip_read_buffer.argtypes = [vp, vp, vp, vp, C.c_size_t]
    lib.argus_hip_copy_slice.argtypes = [vp, vp, vp, vp, C.c_size_t]
    lib.argus_hip_synchronize.argtypes = [vp, vp]
    lib.argus_hip_attention_gen.argtypes = [vp, C.POINTER(AttentionGenArgs)]
    lib.argus_hip_attention_gen_noalloc.argtypes = [vp, C.POINTER(AttentionGenArgs)]
    lib.argus_hip_attention_gen_desc.argtypes = [vp, C.POINTER(AttentionGenArgs), C.POINTER(KvLayoutDesc)]
    lib.argus_hip_flash_attention_prefill.argtypes = [vp, C.POINTER(PrefillArgs)]
    lib.argus_hip_prefill_attention_scores.argtypes = [vp, C.POINTER(PfaArgs)]
    lib.argus_hip_kv_decode_descriptor.argtypes = [vp, vp, C.POINTER(KvLayoutDesc), vp, vp, C.c_int32, C.c_int64]
    lib.argus_hip_kv_encode_descriptor.argtypes = [vp, vp, C.POINTER(KvLayoutDesc), vp, vp, C.c_int64]
    lib.argus_hip_has_quant_attn_kernel.argtypes = [vp, C.c_uint8]
    lib.argus_hip_attention_gen_quant.argtypes = [vp, C.POINTER(QuantAttnArgs)]
    lib.argus_hip_attention_gen_quant_ex.argtypes = [vp, C.POINTER(QuantAttnArgs), C.POINTER(QuantAttnExt)]
    lib.argus_hip_gather_update_quant.argtypes = [vp, C.POINTER(QuantGatherArgs)]
    lib.argus_hip_quant_flush.argtypes = [vp, C.POINTER(QuantFlushArgs)]
    lib.argus_hip_quant_dequant_flush.argtypes = [vp, C.POINTER(QuantDequantFlushArgs)]
    lib.argus_hip_quant_scatter_residual.argtypes = [vp, C.POINTER(QuantScatterResidualArgs)]
    lib.argus_hip_score_reduce.argtypes = [vp, C.POINTER(ScoreReduceArgs)]
    lib.argus_hip_score_reduce_per_layer.argtypes = [vp, C.POINTER(ScoreReduceArgs)]
    lib.argus_hip_score_reduce_ex.argtypes = [vp, C.POINTER(ScoreReduceArgs), C.POINTER(ScoreReduceExt)]
    lib.argus_hip_score_reduce_per_layer_ex.argtypes = [vp, C.POINTER(ScoreReduceArgs), C.POINTER(ScoreReduceExt)]
    sc16 = [vp, vp, vp, vp, vp, vp, i32, i32, i32, i32]
    lib.argus_hip_kv_scatter_f32_to_f16.argtypes = sc16
    lib.argus_hip_kv_scatter_f32_to_f16_batch.argtypes = sc16 + [i32]
    lib.argus_hip_kv_scatter_f32_batch.argtypes = sc16 + [i32]
    lib.argus_hip_quant_requant.argtypes = [vp, C.POINTER(QuantRequantArgs)]
    lib.argus_hip_quant_cache_make.argtypes = [C.POINTER(QuantCacheMakeArgs)]
    for name in ("current_pos", "capacity", "current_bits", "flush_if_full", "drop"):
        getattr(lib, "argus_hip_quant_cache_" + name).argtypes = [vp]
    lib.argus_hip_quant_cache_update.argtypes = [vp, C.POINTER(QuantCacheUpdateArgs)]
    lib.argus_hip_quant_cache_assemble_view.argtypes = [vp, C.POINTER(QuantCacheViewOut)]
    lib.argus_hip_quant_cache_get_raw_buffers.argtypes = [vp, C.POINTER(QuantCacheRawBuffersOut)]
    lib.argus_hip_quant_cache_transition_bits.argtypes = [vp, C.c_uint8]
    lib.argus_hip_quant_cache_get_vtable.argtypes = []
    for name in EXPORTED_SYMBOLS:
        if name != "argus_hip_last_error":
            getattr(lib, name).restype = C.c_int
    lib.argus_hip_quant_attn_cap_make.argtypes = [C.POINTER(QuantAttnMakeArgs)]
    lib.argus_hip_quant_attn_cap_make.restype = vp
    lib.argus_hip_quant_attn_cap_drop.argtypes = [vp]
    lib.argus_hip_quant_attn_cap_drop.restype = None
    lib.argus_hip_quant_attn_cap_has_kernel.argtypes = [vp, C.c_uint8]
    lib.argus_hip_quant_attn_cap_has_kernel.restype = C.c_bool
    lib.argus_hip_quant_attn_cap_is_nosub_device.argtypes = [vp]
    lib.argus_hip_quant_attn_cap_is_nosub_device.restype = C.c_bool
    lib.argus_hip_quant_attn_cap_attention_gen_quant.argtypes = [vp, C.POINTER(QuantAttnArgs)]
    lib.argus_hip_quant_attn_cap_gather_update_quant.argtypes = [vp, C.POINTER(QuantGatherArgs)]
    lib.argus_hip_quant_attn_cap_dequant_flush.argtypes = [vp, C.POINTER(QuantDequantFlushArgs)]
    lib.argus_hip_quant_attn_cap_scatter_residual.argtypes = [vp, C.POINTER(QuantScatterResidualArgs)]
    lib.argus_hip_quant_attn_get_vtable.argtypes = []
    lib.argus_hip_quant_attn_get_vtable.restype = C.POINTER(QuantAttnVTable)
    lib.register_backend_caps_v2.argtypes = []
    lib.register_backend_caps_v2.restype = BackendCapExportAbi
    lib.argus_hip_quant_cache_make.restype = vp
    lib.argus_hip_quant_cache_get_vtable.restype = C.POINTER(QuantCacheVTable)
    lib.argus_hip_quant_cache_current_pos.restype = C.c_size_t
    lib.argus_hip_quant_cache_capacity.restype = C.c_size_t
    lib.argus_hip_quant_cache_current_bits.restype = C.c_uint8
    lib.argus_hip_quant_cache_get_raw_buffers.restype = C.c_bool
    lib.argus_hip_quant_cache_drop.restype = None


_bind()


class QuantCache:
    """Handle of argus_hip_quant_cache_* (QuantCacheBackend, crates/argus-extension-api/src/lib.rs:2017-2035)."""

    def __init__(self, ctx, handle):
        self.ctx, self.handle = ctx, C.c_void_p(handle)

    def close(self):
        if self.handle:
            lib.argus_hip_quant_cache_drop(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def current_pos(self):
        return lib.argus_hip_quant_cache_current_pos(self.handle)

    def capacity(self):
        return lib.argus_hip_quant_cache_capacity(self.handle)

    def current_bits(self):
        return lib.argus_hip_quant_cache_current_bits(self.handle)

    def update(self, k, v, check=True):
        """k, v: device F32 [seq_len, kv_heads, head_dim]."""
        a = QuantCacheUpdateArgs(stream=_stream(), k_in_mem=_ptr(k), v_in_mem=_ptr(v), seq_len=k.shape[0])
        return self.ctx._check(lib.argus_hip_quant_cache_update(self.handle, C.byref(a)), check)

    def flush_if_full(self, check=True):
        return self.ctx._check(lib.argus_hip_quant_cache_flush_if_full(self.handle), check)

    def assemble_view(self):
        out = QuantCacheViewOut()
        self.ctx._check(lib.argus_hip_quant_cache_assemble_view(self.handle, C.byref(out)))
        return out

    def get_raw_buffers(self):
        out = QuantCacheRawBuffersOut()
        return out if lib.argus_hip_quant_cache_get_raw_buffers(self.handle, C.byref(out)) else None

    def transition_bits(self, bits, check=True):
        return self.ctx._check(lib.argus_hip_quant_cache_transition_bits(self.handle, bits), check)


class ArgusHipError(RuntimeError):
    def __init__(self, code, msg):
        super().__init__("argus_hip rc=%d: %s" % (code, msg))
        self.code = code


def _ptr(t):
    return 0 if t is None else t.data_ptr()


def _stream():
    import torch
    return torch.cuda.current_stream().cuda_stream


def _kv_dtype(t):
    import torch
    if t.dtype == torch.float16:
        return F16
    if t.dtype == torch.float32:
        return F32
    raise TypeError("unsupported KV dtype %s" % t.dtype)


class Context:
    """Owns one argus_hip_ctx.  Methods take torch CUDA tensors and return the C return code
    (raising ArgusHipError on a negative one unless check=False)."""

    def __init__(self, device=0, max_batch=0, max_heads_q=0, max_head_dim=0, max_seq_len=0):
        h = C.c_void_p()
        if max_batch or max_heads_q or max_head_dim or max_seq_len:
            opts = CreateOpts(max_batch, max_heads_q, max_head_dim, max_seq_len)
            rc = lib.argus_hip_create_ex(device, C.byref(opts), C.byref(h))
        else:
            rc = lib.argus_hip_create(device, C.byref(h))
        if rc != OK:
            raise ArgusHipError(rc, "argus_hip_create failed (no HIP device?)")
        self.handle = h

    def close(self):
        if self.handle:
            lib.argus_hip_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def last_error(self):
        return lib.argus_hip_last_error(self.handle).decode()

    def _check(self, rc, check=True):
        if rc < 0 and check:
            raise ArgusHipError(rc, self.last_error())
        return rc

    def device_info(self):
        info = DeviceInfo()
        self._check(lib.argus_hip_get_device_info(self.handle, C.byref(info)))
        return info

    def kernel_timing_begin(self, max_launches):
        self._check(lib.argus_hip_kernel_timing_begin(self.handle, max_launches))

    def kernel_timing_end(self, capacity=4096):
        """Per-launch durations (ms) of the dominant kernel since kernel_timing_begin."""
        buf = (C.c_float * capacity)()
        n = C.c_int32(0)
        self._check(lib.argus_hip_kernel_timing_end(self.handle, buf, capacity, C.byref(n)))
        return [buf[i] for i in range(min(n.value, capacity))]

    def kernel_timing_end2(self, capacity=4096):
        """(dominant-kernel ms, tail ms) per call: the tail is the combine pass of a split-KV decode."""
        buf, tail = (C.c_float * capacity)(), (C.c_float * capacity)()
        n = C.c_int32(0)
        self._check(lib.argus_hip_kernel_timing_end2(self.handle, buf, tail, capacity, C.byref(n)))
        m = min(n.value, capacity)
        return [buf[i] for i in range(m)], [tail[i] for i in range(m)]

    def last_decode_plan(self):
        p = DecodePlan()
        self._check(lib.argus_hip_last_decode_plan(self.handle, C.byref(p)))
        return {f: getattr(p, f) for f, _ in DecodePlan._fields_}

    def reserve_workspace(self, nbytes):
        return self._check(lib.argus_hip_reserve_workspace(self.handle, nbytes))

    def buffer_shift(self, t, src_offset, dst_offset, count, check=True):
        """Backend::buffer_shift: move `count` elements inside tensor `t` (memmove semantics)."""
        es = t.element_size()
        base = t.data_ptr()
        return self._check(lib.argus_hip_buffer_shift(self.handle, _stream(), base + dst_offset * es, base + src_offset * es,
                                                      count * es), check)

    def copy_slice(self, dst, src, nbytes, check=True):
        return self._check(lib.argus_hip_copy_slice(self.handle, _stream(), dst, src, nbytes), check)

    def write_buffer_range(self, t, dst_offset_bytes, host_array, check=True):
        return self._check(lib.argus_hip_write_buffer_range(self.handle, _stream(), t.data_ptr(), dst_offset_bytes,
                                                            host_array.ctypes.data, host_array.nbytes), check)

    # -- (a-1) ---------------------------------------------------------------------------
    def attention_gen(self, q, k, v, out, num_heads_kv, cache_seq_len, capacity=0,
                      layout=HEAD_MAJOR, scores=None, score_stride=0, kv_index=None, kv_start=0,
                      batch=1, kv_batch_stride=0, index_batch_stride=0, softcap=0.0, scale=0.0,
                      check=True, kv_dtype=None, noalloc=False, desc=None, score_stats=None):
        """q/out [batch, Hq, d] (or [Hq, d]) f32; k/v device caches; scores [batch, Hq, stride].
        kv_dtype: Q4_0 / Q4_1 / Q8_0 / Q2_0 for uint8 tensors of blocks (default: from the tensor dtype).
        noalloc: go through argus_hip_attention_gen_noalloc (partials in the library's static array).
        desc: KVLayoutDesc tuple of a uint8 cache of blocks: go through argus_hip_attention_gen_desc.
        score_stats [batch, Hq, 2] f32: `scores` keeps the logits, (max, sum) of every row go here."""
        hq, d = q.shape[-2], q.shape[-1]
        a = AttentionGenArgs(
            stream=_stream(), q=_ptr(q), k_cache=_ptr(k), v_cache=_ptr(v), out=_ptr(out),
            scores_out=_ptr(scores), kv_index=_ptr(kv_index), num_heads_q=hq,
            num_heads_kv=num_heads_kv, head_dim=d, cache_seq_len=cache_seq_len, capacity=capacity,
            kv_start=kv_start, layout=layout,
            kv_dtype=0 if desc is not None else _kv_dtype(k) if kv_dtype is None else kv_dtype,
            batch=batch, score_stride=score_stride, q_batch_stride=0, out_batch_stride=0,
            kv_batch_stride=kv_batch_stride, score_batch_stride=0,
            index_batch_stride=index_batch_stride, softcap=softcap, scale=scale,
            score_stats=_ptr(score_stats), stats_batch_stride=0)
        if desc is not None:
            dd = KvLayoutDesc(*desc)
            return self._check(lib.argus_hip_attention_gen_desc(self.handle, C.byref(a), C.byref(dd)), check)
        fn = lib.argus_hip_attention_gen_noalloc if noalloc else lib.argus_hip_attention_gen
        return self._check(fn(self.handle, C.byref(a)), check)

    # -- (a-2) ---------------------------------------------------------------------------
    def flash_attention_prefill(self, q, k, v, out, n_heads_q, n_heads_kv, seq_len, cache_seq_len,
                                head_dim, kv_capacity, batch_size=1, is_head_major=True, window=0,
                                check=True):
        a = PrefillArgs(
            stream=_stream(), q=_ptr(q), k_cache=_ptr(k), v_cache=_ptr(v), out=_ptr(out),
            n_heads_q=n_heads_q, n_heads_kv=n_heads_kv, seq_len=seq_len,
            cache_seq_len=cache_seq_len, head_dim=head_dim, kv_capacity=kv_capacity,
            batch_size=batch_size, is_head_major=int(is_head_major), q_dtype=_kv_dtype(q),
            kv_dtype=_kv_dtype(k), out_dtype=_kv_dtype(out), window=window)
        return self._check(lib.argus_hip_flash_attention_prefill(self.handle, C.byref(a)), check)

    # -- (a-6) ---------------------------------------------------------------------------
    def prefill_attention_scores(self, q, k, n_heads_q, n_heads_kv, head_dim, seq_len, cache_seq_len,
                                 k_pos_stride, kv_head_stride, q_start_pos, q_window, window=None,
                                 sum_out=None, per_row=None, per_head=False, check=True):
        a = PfaArgs(stream=_stream(), q=_ptr(q), k=_ptr(k), k_dtype=_kv_dtype(k), n_heads_q=n_heads_q,
                    n_heads_kv=n_heads_kv, head_dim=head_dim, seq_len=seq_len,
                    cache_seq_len=cache_seq_len, k_pos_stride=k_pos_stride,
                    kv_head_stride=kv_head_stride, q_start_pos=q_start_pos, q_window=q_window,
                    has_window=0 if window is None else 1, window=0 if window is None else window,
                    sum_out=_ptr(sum_out) if sum_out is not None else None,
                    per_row_out=_ptr(per_row) if per_row is not None else None,
                    per_row_per_head=1 if per_head else 0)
        return self._check(lib.argus_hip_prefill_attention_scores(self.handle, C.byref(a)), check)

    # -- (a-3) ---------------------------------------------------------------------------
    def has_quant_attn_kernel(self, bits):
        return lib.argus_hip_has_quant_attn_kernel(self.handle, bits) == 1

    def attention_gen_quant(self, q, qk, qv, res_k, res_v, out, num_heads_kv, q_tokens, res_tokens,
                            res_cap, scale, bits, scores_host=None, scores_dev=None,
                            score_stride=0, softcap=0.0, batch=1, block_batch_stride_bytes=0,
                            res_batch_stride=0, check=True, score_stats=None):
        """scores_host: numpy float32 array (host readback, reference contract);
        scores_dev: torch tensor (device)."""
        import torch
        hq, d = q.shape[-2], q.shape[-1]
        a = QuantAttnArgs(
            stream=_stream(), q_mem=_ptr(q), qk_mem=_ptr(qk), qv_mem=_ptr(qv),
            res_k_mem=_ptr(res_k), res_v_mem=_ptr(res_v), out_mem=_ptr(out),
            scores_out=(scores_host.ctypes.data if scores_host is not None else None),
            scores_len=(scores_host.size if scores_host is not None else 0), num_heads_q=hq,
            num_heads_kv=num_heads_kv, head_dim=d, q_tokens=q_tokens, res_tokens=res_tokens,
            res_cap=res_cap, scale=scale, bits=bits)
        res_dtype = F16 if res_k.dtype == torch.float16 else F32
        if scores_dev is None and res_dtype == F32 and softcap == 0.0 and batch == 1 and score_stats is None:
            return self._check(lib.argus_hip_attention_gen_quant(self.handle, C.byref(a)), check)
        e = QuantAttnExt(scores_dev=_ptr(scores_dev), score_stride=score_stride,
                         res_dtype=res_dtype, softcap=softcap, batch=batch,
                         block_batch_stride_bytes=block_batch_stride_bytes,
                         res_batch_stride=res_batch_stride, score_batch_stride=0,
                         score_stats_dev=_ptr(score_stats) or 0)
        return self._check(lib.argus_hip_attention_gen_quant_ex(self.handle, C.byref(a), C.byref(e)), check)

    def gather_update_quant(self, inp, residual, kv_heads, res_cap, head_dim, seq_len, res_pos,
                            check=True):
        a = QuantGatherArgs(stream=_stream(), input_mem=_ptr(inp), residual_mem=_ptr(residual),
                            kv_heads=kv_heads, res_cap=res_cap, head_dim=head_dim, seq_len=seq_len,
                            res_pos=res_pos)
        return self._check(lib.argus_hip_gather_update_quant(self.handle, C.byref(a)), check)

    def quant_flush(self, res_k, res_v, qk, qv, kv_heads, res_cap, head_dim, flush_tokens,
                    k_block_start, v_block_start, bits, check=True, out_res_cap=0):
        a = QuantFlushArgs(stream=_stream(), res_k_mem=_ptr(res_k), res_v_mem=_ptr(res_v),
                           qk_mem=_ptr(qk), qv_mem=_ptr(qv), kv_heads=kv_heads, res_cap=res_cap,
                           head_dim=head_dim, flush_tokens=flush_tokens,
                           k_block_start=k_block_start, v_block_start=v_block_start, bits=bits,
                           out_res_cap=out_res_cap)
        return self._check(lib.argus_hip_quant_flush(self.handle, C.byref(a)), check)

    def quant_requant(self, src, dst, n_blocks, old_bits, new_bits, check=True):
        a = QuantRequantArgs(stream=_stream(), src_mem=_ptr(src), dst_mem=_ptr(dst), n_blocks=n_blocks,
                             old_bits=old_bits, new_bits=new_bits)
        return self._check(lib.argus_hip_quant_requant(self.handle, C.byref(a)), check)

    def quant_cache(self, kv_heads, head_dim, max_seq_len, residual_size, bits):
        """The KIVI container behind the CACHE-category vtable; None when `make` refuses."""
        a = QuantCacheMakeArgs(ctx=self.handle, device=None, stream=_stream(), build_opts=None, kv_heads=kv_heads,
                               head_dim=head_dim, max_seq_len=max_seq_len, residual_size=residual_size, bits=bits)
        h = lib.argus_hip_quant_cache_make(C.byref(a))
        return QuantCache(self, h) if h else None

    def quant_dequant_flush(self, blocks, attn, kv_heads, head_dim, n_groups_or_tokens, tok_base,
                            block_start, bits, is_key, check=True):
        a = QuantDequantFlushArgs(stream=_stream(), q_blocks_mem=_ptr(blocks), attn_mem=_ptr(attn),
                                  kv_heads=kv_heads, head_dim=head_dim,
                                  n_groups_or_tokens=n_groups_or_tokens, tok_base=tok_base,
                                  block_start=block_start, bits=bits, is_key=1 if is_key else 0)
        return self._check(lib.argus_hip_quant_dequant_flush(self.handle, C.byref(a)), check)

    def quant_scatter_residual(self, residual, attn, kv_heads, res_cap, head_dim, res_pos, tok_base,
                               check=True):
        a = QuantScatterResidualArgs(stream=_stream(), res_mem=_ptr(residual), attn_mem=_ptr(attn),
                                     kv_heads=kv_heads, res_cap=res_cap, head_dim=head_dim,
                                     res_pos=res_pos, tok_base=tok_base)
        return self._check(lib.argus_hip_quant_scatter_residual(self.handle, C.byref(a)), check)

    # -- (f-4) ---------------------------------------------------------------------------
    def kv_decode_descriptor(self, desc, src, dst, n_elems, check=True):
        d = KvLayoutDesc(*desc)
        return self._check(lib.argus_hip_kv_decode_descriptor(self.handle, _stream(), C.byref(d), _ptr(src), _ptr(dst),
                                                              _kv_dtype(dst), n_elems), check)

    def kv_encode_descriptor(self, desc, src, dst, n_elems, check=True):
        d = KvLayoutDesc(*desc)
        return self._check(lib.argus_hip_kv_encode_descriptor(self.handle, _stream(), C.byref(d), _ptr(src), _ptr(dst),
                                                              n_elems), check)

    # -- (a-4) ---------------------------------------------------------------------------
    def _score_args(self, scores, importance, head_importance, decay_factor, n_layers, n_heads_q,
                    n_kv_heads, cache_seq_len, score_stride, max_seq_len, layer_flat):
        return ScoreReduceArgs(
            stream=_stream(), score_buf=_ptr(scores), importance=_ptr(importance),
            head_importance=_ptr(head_importance), decay_factor=decay_factor, n_layers=n_layers,
            n_heads_q=n_heads_q, n_kv_heads=n_kv_heads, cache_seq_len=cache_seq_len,
            score_stride=score_stride, max_seq_len=max_seq_len,
            layer_flat_importance=_ptr(layer_flat))

    def score_reduce(self, scores, importance, head_importance, decay_factor, n_layers, n_heads_q,
                     n_kv_heads, cache_seq_len, score_stride, max_seq_len, check=True, stats=None):
        """stats [n_layers, n_heads_q, 2]: `scores` holds logits, normalised while they are read."""
        a = self._score_args(scores, importance, head_importance, decay_factor, n_layers, n_heads_q,
                             n_kv_heads, cache_seq_len, score_stride, max_seq_len, None)
        if stats is not None:
            e = ScoreReduceExt(stats=_ptr(stats))
            return self._check(lib.argus_hip_score_reduce_ex(self.handle, C.byref(a), C.byref(e)), check)
        return self._check(lib.argus_hip_score_reduce(self.handle, C.byref(a)), check)

    def score_reduce_per_layer(self, scores, layer_flat, decay_factor, n_layers, n_heads_q,
                               n_kv_heads, cache_seq_len, score_stride, max_seq_len, check=True, stats=None):
        a = self._score_args(scores, None, None, decay_factor, n_layers, n_heads_q, n_kv_heads,
                             cache_seq_len, score_stride, max_seq_len, layer_flat)
        if stats is not None:
            e = ScoreReduceExt(stats=_ptr(stats))
            return self._check(lib.argus_hip_score_reduce_per_layer_ex(self.handle, C.byref(a), C.byref(e)), check)
        return self._check(lib.argus_hip_score_reduce_per_layer(self.handle, C.byref(a)), check)

    # -- (f-1) ---------------------------------------------------------------------------
    def kv_scatter(self, k_src, v_src, k_dst, v_dst, kv_heads, head_dim, capacity, write_pos,
                   seq_len=None, check=True):
        import torch
        args = [self.handle, _stream(), _ptr(k_src), _ptr(v_src), _ptr(k_dst), _ptr(v_dst),
                kv_heads, head_dim, capacity, write_pos]
        if k_dst.dtype == torch.float32:
            rc = lib.argus_hip_kv_scatter_f32_batch(*args, 1 if seq_len is None else seq_len)
        elif seq_len is None:
            rc = lib.argus_hip_kv_scatter_f32_to_f16(*args)
        else:
            rc = lib.argus_hip_kv_scatter_f32_to_f16_batch(*args, seq_len)
        return self._check(rc, check)
