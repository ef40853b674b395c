"""ctypes loader for the CPU oracle (oracle/argus_oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py.  The product package never imports this module.
Each wrapper takes / returns numpy arrays and forwards to the C restatement of
the reference function named in argus_oracle.c.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libargus_oracle.so")


def build(force=False):
    """Compile libargus_oracle.so with the committed Makefile."""
    if force:
        subprocess.check_call(["make", "-C", _HERE, "clean"], stdout=subprocess.DEVNULL)
    subprocess.check_call(["make", "-C", _HERE], stdout=subprocess.DEVNULL)


def _load():
    if not os.path.exists(_LIB_PATH):
        build()
    return C.CDLL(_LIB_PATH)


_lib = _load()

_f32p = C.POINTER(C.c_float)
_u8p = C.POINTER(C.c_uint8)
_u16p = C.POINTER(C.c_uint16)
_i32p = C.POINTER(C.c_int32)


def _p(a, t=C.c_void_p):
    if a is None:
        return None
    assert a.flags["C_CONTIGUOUS"], "oracle wrappers need contiguous arrays"
    return a.ctypes.data_as(t)


def _sig(name, restype, argtypes):
    fn = getattr(_lib, name)
    fn.restype = restype
    fn.argtypes = argtypes
    return fn


_gen_data = _sig("oracle_gen_data", None, [_f32p, C.c_int64, C.c_uint32])
_f2h = _sig("oracle_f32_to_f16", None, [_f32p, _u16p, C.c_int64])
_attn_scalar = _sig("oracle_attention_gen_scalar", C.c_int, [
    _f32p, C.c_void_p, C.c_void_p, _f32p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int,
    C.c_int, _f32p, C.c_int64, C.c_float, _i32p])
_attn_avx2 = _sig("oracle_attention_gen_avx2", C.c_int, [
    _f32p, C.c_void_p, C.c_void_p, _f32p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int,
    C.c_int, _f32p, C.c_int64, C.c_int])
_flash_strided = _sig("oracle_flash_attention_forward_strided", None, [
    _f32p, _f32p, _f32p, _f32p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int64, C.c_int64,
    C.c_int64, C.c_int64, C.c_int64, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int])
_prefill = _sig("oracle_prefill_attention", C.c_int, [
    _f32p, C.c_void_p, C.c_void_p, _f32p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int,
    C.c_int, C.c_int, C.c_int, C.c_int])
_kq = _sig("oracle_kivi_quantize_block", C.c_int, [_f32p, C.c_int, _u8p])
_kdq = _sig("oracle_kivi_dequantize_block", C.c_int, [_u8p, C.c_int, _f32p])
_krequant = _sig("oracle_kivi_requant", C.c_int, [_u8p, _u8p, C.c_int64, C.c_int, C.c_int])
_kbuild = _sig("oracle_kivi_build", C.c_int, [
    _f32p, _f32p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, _u8p, _u8p, _f32p, _f32p,
    C.POINTER(C.c_int), C.POINTER(C.c_int)])
_kview = _sig("oracle_kivi_assemble_view", C.c_int, [
    _u8p, _u8p, _f32p, _f32p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, _f32p, _f32p])
_kattn = _sig("oracle_kivi_attention", C.c_int, [
    _f32p, _u8p, _u8p, _f32p, _f32p, _f32p, _f32p, C.c_int64, C.c_int, C.c_int, C.c_int, C.c_int,
    C.c_int, C.c_int, C.c_float, C.c_int])
_sbegin = _sig("oracle_score_begin_step", None, [_f32p, _f32p, _f32p, _f32p, C.c_int, C.c_int, C.c_float])
_sacc = _sig("oracle_score_accumulate_layer_gqa", None, [
    _f32p, C.c_int64, C.c_int, C.c_int, C.c_int, C.c_int, _f32p, _f32p, C.c_int])
_send = _sig("oracle_score_end_step", None, [_f32p, _f32p, _f32p, _f32p, C.c_int, C.c_int])
_sfused = _sig("oracle_score_fused_reduce", C.c_int, [
    _f32p, _f32p, _f32p, C.c_float, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int64, C.c_int])
_slayer = _sig("oracle_score_reduce_per_layer", None, [
    _f32p, _f32p, C.c_float, C.c_int, C.c_int, C.c_int, C.c_int64, C.c_int])
_keep = _sig("oracle_compile_keep_top_k", C.c_int, [C.c_int, C.c_int, C.c_int, C.c_int, _f32p, _i32p])
_skeep = _sig("oracle_streaming_keep", C.c_int, [C.c_int, C.c_int, C.c_int, C.c_int, _i32p])
_compact = _sig("oracle_compact_keep", None, [
    C.c_void_p, C.c_void_p, _i32p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int])
_pfa = _sig("oracle_prefill_attention_scores", C.c_int, [
    _f32p, _f32p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int64, C.c_int64, C.c_int, C.c_int,
    C.c_int, _f32p, _f32p, C.c_int])
_desc_bb = _sig("oracle_desc_block_bytes", C.c_int, [C.c_int, C.c_int, C.c_int])
_desc_dec = _sig("oracle_decode_via_descriptor", C.c_int, [C.c_int, C.c_int, C.c_int, C.c_int, _u8p, _f32p, C.c_int64])
_desc_enc = _sig("oracle_encode_via_descriptor", C.c_int, [C.c_int, C.c_int, C.c_int, C.c_int, _f32p, _u8p, C.c_int64])
_scatter = _sig("oracle_kv_scatter", None, [
    _f32p, _f32p, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int])

KV_F32, KV_F16 = 0, 1


def gen_data(n, seed):
    """The reference tests' LCG in [-1, 1)."""
    out = np.empty(n, np.float32)
    _gen_data(_p(out, _f32p), n, seed & 0xFFFFFFFF)
    return out


def f32_to_f16_bits(x):
    x = np.ascontiguousarray(x, np.float32)
    out = np.empty(x.shape, np.uint16)
    _f2h(_p(x, _f32p), _p(out, _u16p), x.size)
    return out


def _kv_dtype(k):
    if k.dtype == np.float32:
        return KV_F32
    if k.dtype in (np.float16, np.uint16):
        return KV_F16
    raise TypeError(k.dtype)


def attention_gen(q, k, v, n_heads_kv, cache_seq_len, capacity, head_major=True, scores=False,
                  scores_stride=None, impl="scalar", softcap=0.0, kv_index=None, n_threads=0):
    """Backend::attention_gen on the CPU.  q [Hq, d] f32; k, v flat or shaped caches."""
    q = np.ascontiguousarray(q, np.float32)
    hq, d = q.shape
    out = np.zeros((hq, d), np.float32)
    stride = scores_stride if scores_stride is not None else cache_seq_len
    sc = np.zeros((hq, stride), np.float32) if scores else None
    kd = _kv_dtype(k)
    if impl == "scalar":
        ki = None if kv_index is None else np.ascontiguousarray(kv_index, np.int32)
        rc = _attn_scalar(_p(q, _f32p), _p(k), _p(v), _p(out, _f32p), hq, n_heads_kv, d,
                          cache_seq_len, capacity, int(head_major), kd, _p(sc, _f32p), stride,
                          float(softcap), _p(ki, _i32p))
    else:
        assert softcap == 0.0 and kv_index is None, "AVX2 path mirrors the reference: no extras"
        rc = _attn_avx2(_p(q, _f32p), _p(k), _p(v), _p(out, _f32p), hq, n_heads_kv, d,
                        cache_seq_len, capacity, int(head_major), kd, _p(sc, _f32p), stride,
                        n_threads)
    if rc != 0:
        raise ValueError("oracle attention_gen rc=%d" % rc)
    return (out, sc) if scores else out


def flash_attention_forward_strided(q, k, v, n_heads_q, n_heads_kv, q_len, kv_len, head_dim,
                                    q_stride, k_stride, v_stride, out_stride, kv_head_stride,
                                    q_start_pos, br=32, bc=32, window=0, n_threads=0):
    q = np.ascontiguousarray(q, np.float32)
    k = np.ascontiguousarray(k, np.float32)
    v = np.ascontiguousarray(v, np.float32)
    out = np.zeros(q_len * out_stride, np.float32)
    _flash_strided(_p(q, _f32p), _p(k, _f32p), _p(v, _f32p), _p(out, _f32p), n_heads_q, n_heads_kv,
                   q_len, kv_len, head_dim, q_stride, k_stride, v_stride, out_stride,
                   kv_head_stride, q_start_pos, br, bc, window or 0, n_threads)
    return out


def prefill_attention(q, k, v, n_heads_kv, cache_seq_len, capacity, window=0, n_threads=0):
    """StandardFormat::prefill_attention CPU arm.  q [B, S, Hq, d] f32; k, v [B, Hkv, cap, d]."""
    q = np.ascontiguousarray(q, np.float32)
    b, s, hq, d = q.shape
    out = np.zeros_like(q)
    rc = _prefill(_p(q, _f32p), _p(k), _p(v), _p(out, _f32p), hq, n_heads_kv, s, cache_seq_len, d,
                  capacity, b, _kv_dtype(k), window or 0, n_threads)
    if rc != 0:
        raise ValueError("oracle prefill rc=%d" % rc)
    return out


def kivi_block_bytes(bits):
    return 4 + 32 * bits // 8


def kivi_quantize_block(src, bits):
    src = np.ascontiguousarray(src, np.float32)
    assert src.size == 32
    dst = np.zeros(kivi_block_bytes(bits), np.uint8)
    assert _kq(_p(src, _f32p), bits, _p(dst, _u8p)) == 0
    return dst


def kivi_dequantize_block(blk, bits):
    blk = np.ascontiguousarray(blk, np.uint8)
    out = np.zeros(32, np.float32)
    assert _kdq(_p(blk, _u8p), bits, _p(out, _f32p)) == 0
    return out


def kivi_requant(blocks, old_bits, new_bits):
    """transition_bits between two quantised widths on a uint8 block stream: every block dequantised
    and quantised again at the new width, order kept (quant_window_cache.rs:1350-1362)."""
    blocks = np.ascontiguousarray(blocks, np.uint8)
    n = blocks.size // kivi_block_bytes(old_bits)
    out = np.zeros(n * kivi_block_bytes(new_bits), np.uint8)
    if _krequant(_p(blocks, _u8p), _p(out, _u8p), n, old_bits, new_bits) != 0:
        raise ValueError("oracle kivi_requant: bits %d -> %d" % (old_bits, new_bits))
    return out


def kivi_build(k_tokens, v_tokens, res_cap, bits):
    """Replay token-by-token appends through the KIVI container.

    k_tokens, v_tokens: [T, Hkv, d] f32.  Returns dict(qk, qv, res_k, res_v, q_tokens,
    res_tokens) with qk/qv as uint8 block streams in device order.
    """
    k_tokens = np.ascontiguousarray(k_tokens, np.float32)
    v_tokens = np.ascontiguousarray(v_tokens, np.float32)
    t, hkv, d = k_tokens.shape
    bb = kivi_block_bytes(bits)
    max_flush = t // res_cap
    nblk = max(1, max_flush * hkv * res_cap * d // 32)
    qk = np.zeros(nblk * bb, np.uint8)
    qv = np.zeros(nblk * bb, np.uint8)
    res_k = np.zeros((hkv, res_cap, d), np.float32)
    res_v = np.zeros((hkv, res_cap, d), np.float32)
    qt, rt = C.c_int(0), C.c_int(0)
    rc = _kbuild(_p(k_tokens, _f32p), _p(v_tokens, _f32p), t, hkv, d, res_cap, bits, _p(qk, _u8p),
                 _p(qv, _u8p), _p(res_k, _f32p), _p(res_v, _f32p), C.byref(qt), C.byref(rt))
    if rc != 0:
        raise ValueError("oracle kivi_build rc=%d" % rc)
    used = qt.value * hkv * d // 32 * bb
    return dict(qk=qk[:max(used, 1)].copy() if used else qk[:bb].copy(),
                qv=qv[:max(used, 1)].copy() if used else qv[:bb].copy(),
                res_k=res_k, res_v=res_v, q_tokens=qt.value, res_tokens=rt.value,
                res_cap=res_cap, bits=bits, kv_heads=hkv, head_dim=d)


def kivi_assemble_view(c):
    total = c["q_tokens"] + c["res_tokens"]
    hkv, d = c["kv_heads"], c["head_dim"]
    ak = np.zeros((max(total, 1), hkv, d), np.float32)
    av = np.zeros((max(total, 1), hkv, d), np.float32)
    rc = _kview(_p(c["qk"], _u8p), _p(c["qv"], _u8p), _p(c["res_k"], _f32p), _p(c["res_v"], _f32p),
                c["q_tokens"], c["res_tokens"], hkv, d, c["res_cap"], c["bits"], _p(ak, _f32p),
                _p(av, _f32p))
    if rc != 0:
        raise ValueError("oracle kivi_assemble_view rc=%d" % rc)
    return ak[:total], av[:total]


def kivi_dequant_flush_f16(blocks, attn, kv_heads, head_dim, n_groups_or_tokens, tok_base, block_start,
                           bits, is_key):
    """F16-view dequant of one flush (crates/techniques/kivi/src/kivi_q2.cu:18-92, generalised from
    Q2 to the 4- and 8-bit codecs): attn is [max_seq, kv_heads, head_dim] float16, written in place.
    Keys: block (h, g, ch) -> tokens tok_base + 32 g + i of channel ch; values: block (h, t, b) ->
    channels 32 b + i of token tok_base + t.  out = f16(code * d + m) in float32."""
    bb = kivi_block_bytes(bits)
    blocks = np.ascontiguousarray(blocks, np.uint8).reshape(-1, bb)
    n = n_groups_or_tokens
    nblk = kv_heads * n * (head_dim if is_key else head_dim // 32)
    blk = blocks[block_start:block_start + nblk]
    d = blk[:, 0:2].copy().view(np.float16).astype(np.float32)      # [nblk, 1]
    m = blk[:, 2:4].copy().view(np.float16).astype(np.float32)
    qs = blk[:, 4:]
    per = 8 // bits
    idx = np.arange(32)
    codes = (qs[:, idx // per] >> ((idx % per) * bits).astype(np.uint8)) & ((1 << bits) - 1)
    vals = (codes.astype(np.float32) * d + m).astype(np.float16)     # [nblk, 32]
    if is_key:
        v = vals.reshape(kv_heads, n, head_dim, 32)                  # [h, g, ch, i]
        for g in range(n):
            attn[tok_base + 32 * g:tok_base + 32 * g + 32] = v[:, g].transpose(2, 0, 1)
    else:
        v = vals.reshape(kv_heads, n, head_dim // 32, 32)            # [h, t, b, i]
        attn[tok_base:tok_base + n] = v.transpose(1, 0, 2, 3).reshape(n, kv_heads, head_dim)
    return attn


def kivi_scatter_residual_f16(residual, attn, kv_heads, res_cap, head_dim, res_pos, tok_base):
    """kivi_q2.cu:94-116: rows 0..res_pos of the F32 ring [kv_heads, res_cap, head_dim] -> rows
    tok_base.. of the F16 view."""
    r = np.asarray(residual, np.float32).reshape(kv_heads, res_cap, head_dim)
    attn[tok_base:tok_base + res_pos] = r[:, :res_pos].transpose(1, 0, 2).astype(np.float16)
    return attn


def kivi_attention(q, c, scale, scores=False, score_stride=None):
    q = np.ascontiguousarray(q, np.float32)
    hq, d = q.shape
    total = c["q_tokens"] + c["res_tokens"]
    out = np.zeros((hq, d), np.float32)
    stride = score_stride if score_stride is not None else total
    sc = np.zeros((hq, stride), np.float32) if scores else None
    rc = _kattn(_p(q, _f32p), _p(c["qk"], _u8p), _p(c["qv"], _u8p), _p(c["res_k"], _f32p),
                _p(c["res_v"], _f32p), _p(out, _f32p), _p(sc, _f32p), stride, hq, c["kv_heads"], d,
                c["q_tokens"], c["res_tokens"], c["res_cap"], float(scale), c["bits"])
    if rc != 0:
        raise ValueError("oracle kivi_attention rc=%d" % rc)
    return (out, sc) if scores else out


class ScoreProducer:
    """AttnScoreProducer (flat + per-KV-head buffers) on the CPU."""

    def __init__(self, max_seq_len, n_kv_heads, decay=0.0):
        self.max_seq_len, self.n_kv_heads = max_seq_len, n_kv_heads
        self.decay = min(max(decay, 0.0), 1.0)
        self.importance = np.zeros(max_seq_len, np.float32)
        self.head_importance = np.zeros(n_kv_heads * max_seq_len, np.float32)
        self.step = np.zeros(max_seq_len, np.float32)
        self.head_step = np.zeros(n_kv_heads * max_seq_len, np.float32)

    def begin_step(self):
        _sbegin(_p(self.importance, _f32p), _p(self.head_importance, _f32p), _p(self.step, _f32p),
                _p(self.head_step, _f32p), self.max_seq_len, self.n_kv_heads, self.decay)

    def accumulate_layer_gqa(self, scores, stride, cache_seq_len, n_heads_q, score_offset=0):
        scores = np.ascontiguousarray(scores, np.float32)
        _sacc(_p(scores, _f32p), stride, cache_seq_len, n_heads_q, self.n_kv_heads, score_offset,
              _p(self.step, _f32p), _p(self.head_step, _f32p), self.max_seq_len)

    def end_step(self):
        _send(_p(self.importance, _f32p), _p(self.head_importance, _f32p), _p(self.step, _f32p),
              _p(self.head_step, _f32p), self.max_seq_len, self.n_kv_heads)


def score_fused_reduce(scores, importance, head_importance, decay_factor, n_layers, n_heads_q,
                       n_kv_heads, cache_seq_len, score_stride, max_seq_len):
    scores = np.ascontiguousarray(scores, np.float32)
    rc = _sfused(_p(scores, _f32p), _p(importance, _f32p), _p(head_importance, _f32p),
                 float(decay_factor), n_layers, n_heads_q, n_kv_heads, cache_seq_len, score_stride,
                 max_seq_len)
    if rc != 0:
        raise ValueError("oracle score_fused_reduce rc=%d" % rc)


def score_reduce_per_layer(scores, layer_flat, decay_factor, n_layers, n_heads_q, cache_seq_len,
                           score_stride, max_seq_len):
    scores = np.ascontiguousarray(scores, np.float32)
    _slayer(_p(scores, _f32p), _p(layer_flat, _f32p), float(decay_factor), n_layers, n_heads_q,
            cache_seq_len, score_stride, max_seq_len)


def compile_keep_top_k(current, prefix, recent, heavy, score=None):
    keep = np.zeros(max(current, 1), np.int32)
    sc = None if score is None else np.ascontiguousarray(score, np.float32)
    n = _keep(current, prefix, recent, heavy, _p(sc, _f32p), _p(keep, _i32p))
    return keep[:n].copy()


def streaming_keep(sink, window, current, target):
    keep = np.zeros(max(current, 1), np.int32)
    n = _skeep(sink, window, current, target, _p(keep, _i32p))
    return None if n < 0 else keep[:n].copy()


def compact_keep(src, keep, dst_capacity):
    """src HeadMajor [Hkv, cap, d]; gathers kept rows to slots 0..n of a new cache."""
    src = np.ascontiguousarray(src)
    hkv, cap, d = src.shape
    keep = np.ascontiguousarray(keep, np.int32)
    dst = np.zeros((hkv, dst_capacity, d), src.dtype)
    _compact(_p(src), _p(dst), _p(keep, _i32p), len(keep), hkv, cap, dst_capacity, d,
             src.dtype.itemsize)
    return dst


def h2o_keep_spec(current, hh_size, recent_size, protected_prefix=0, importance=None, head_scores=None):
    """H2o::partition + H2o::keep_spec, crates/techniques/h2o/src/lib.rs:118-160.
    Returns None (already within the absolute budget prefix + hh_size + recent_size),
    ("per_head", [keep per KV head]) when per-(kv_head, pos) scores are present, else
    ("layer", keep) from the flat importance, or from recency alone when there are no scores
    (the whole evictable budget hh_size + recent_size goes to the recent window, lib.rs:95-106).
    importance: [>= 0 entries]; positions past its end score 0.0 (`imp.get(pos).unwrap_or(0.0)`).
    head_scores: [n_kv_heads, >= current]."""
    prefix = min(protected_prefix, current)
    if current <= prefix + hh_size + recent_size:
        return None
    if head_scores is not None:
        hs = np.asarray(head_scores, np.float32)
        return "per_head", [compile_keep_top_k(current, prefix, recent_size, hh_size, hs[h, :current]) for h in range(hs.shape[0])]
    if importance is not None:
        imp = np.zeros(current, np.float32)
        n = min(current, len(importance))
        imp[:n] = np.asarray(importance, np.float32)[:n]
        return "layer", compile_keep_top_k(current, prefix, recent_size, hh_size, imp)
    return "layer", compile_keep_top_k(current, prefix, hh_size + recent_size, 0, None)


def keep_batches(keep, write_start=0):
    """The runs KVCache::compact_keep_positions moves (engine/src/kv/kv_cache.rs:1266-1306): consecutive
    source positions merge into one shift; a run already in place is skipped.  Yields (src, dst, count)
    in the order the reference issues them."""
    keep = [int(x) for x in keep]
    if not keep:
        return
    write_pos = write_start
    src0, dst0, count = keep[0], write_pos, 1
    write_pos += 1
    for pos in keep[1:]:
        if pos == src0 + count:
            count += 1
        else:
            if src0 != dst0:
                yield src0, dst0, count
            src0, dst0, count = pos, write_pos, 1
        write_pos += 1
    if src0 != dst0:
        yield src0, dst0, count


def compact_keep_in_place(cache, keep, head=None, write_start=0):
    """compact_keep_positions / compact_keep_positions_for_head on a HeadMajor [Hkv, cap, d] array, in
    place, through the same overlap-safe row shifts (shift_positions, kv_cache.rs:1002-1100: one
    buffer_shift per head and run)."""
    heads = range(cache.shape[0]) if head is None else (head,)
    for src, dst, count in keep_batches(keep, write_start):
        for h in heads:
            cache[h, dst:dst + count] = cache[h, src:src + count].copy()  # memmove
    return cache


def kv_scatter(k_src, v_src, k_dst, v_dst, write_pos_start):
    """kv_scatter_f32_to_f16[_batch] / _f32_batch.  src [S, Hkv, d] f32; dst [Hkv, cap, d]."""
    k_src = np.ascontiguousarray(k_src, np.float32)
    v_src = np.ascontiguousarray(v_src, np.float32)
    s, hkv, d = k_src.shape
    cap = k_dst.shape[1]
    _scatter(_p(k_src, _f32p), _p(v_src, _f32p), _p(k_dst), _p(v_dst), hkv, d, cap,
             write_pos_start, s, int(k_dst.dtype != np.float32))


def prefill_attention_scores(q, k, n_heads_q, n_heads_kv, head_dim, seq_len, cache_seq_len, k_pos_stride,
                             kv_head_stride, q_start_pos, q_window, window=None, sum_out=None,
                             per_row=None, per_head=False):
    """PFA side channel (standard_format.rs:1400-1510).  q [seq_len, n_heads_q, head_dim] f32, k a flat
    f32 array addressed by the strides; sum_out / per_row are float32 arrays updated in place."""
    q = np.ascontiguousarray(q, np.float32)
    k = np.ascontiguousarray(k, np.float32)
    rc = _pfa(_p(q, _f32p), _p(k, _f32p), n_heads_q, n_heads_kv, head_dim, seq_len, cache_seq_len,
              k_pos_stride, kv_head_stride, q_start_pos, q_window, -1 if window is None else window,
              _p(sum_out, _f32p), _p(per_row, _f32p), 1 if per_head else 0)
    if rc != 0:
        raise ValueError("oracle prefill_attention_scores rc=%d" % rc)


# KVLayoutDesc vocabulary (argus-extension-api lib.rs:1111-1159): (block_elems, bits, scale_layout, packing)
SCALE_NONE, SCALE_F16, SCALE_F16_MIN = 0, 1, 2
PACK_DENSE, PACK_NIBBLE, PACK_BYTE, PACK_QUAD = 0, 1, 2, 3
DESC_Q4_0 = (32, 4, SCALE_F16, PACK_NIBBLE)
DESC_Q4_1 = (32, 4, SCALE_F16_MIN, PACK_NIBBLE)
DESC_Q8_0 = (32, 8, SCALE_F16, PACK_BYTE)
DESC_Q2_0 = (32, 2, SCALE_F16_MIN, PACK_QUAD)


def desc_block_bytes(desc):
    return _desc_bb(desc[0], desc[2], desc[3])


def decode_via_descriptor(desc, raw, n_elems):
    """decode_via_descriptor / unpack_block_via_descriptor (format/dtype_layout.rs:102-166, 285-300)."""
    raw = np.ascontiguousarray(raw, np.uint8)
    out = np.zeros(n_elems, np.float32)
    rc = _desc_dec(desc[0], desc[1], desc[2], desc[3], _p(raw, _u8p), _p(out, _f32p), n_elems)
    if rc != 0:
        raise ValueError("oracle decode_via_descriptor rc=%d" % rc)
    return out


def encode_via_descriptor(desc, src):
    """encode_via_descriptor (format/dtype_layout.rs:302-396): q4_0 (PerBlockF16 + Nibble) and q2_0
    (PerBlockF16WithMin + Quad) only; anything else raises like the reference's Err."""
    src = np.ascontiguousarray(src, np.float32).reshape(-1)
    out = np.zeros(src.size // desc[0] * max(desc_block_bytes(desc), 1), np.uint8)
    rc = _desc_enc(desc[0], desc[1], desc[2], desc[3], _p(src, _f32p), _p(out, _u8p), src.size)
    if rc != 0:
        raise ValueError("oracle encode_via_descriptor rc=%d" % rc)
    return out


def attention_gen_blocks(q, k_raw, v_raw, desc, n_heads_kv, cache_seq_len, capacity, head_major=True,
                         scores=False, scores_stride=None, softcap=0.0, kv_index=None):
    """Backend::attention_gen over a block-quantised cache: the Q4_0 arm of the scalar CPU backend
    (backend/cpu/common.rs:676-850: each K / V row is dequantised, then the F32 algorithm with its
    guards runs), which is also what the `--kv-format` floor computes after decoding the whole cache
    (kv/standard_format.rs:538-643).  Restated as exactly that composition: decode_via_descriptor of
    the raw bytes, then the scalar attention_gen on the F32 cache."""
    q = np.ascontiguousarray(q, np.float32)
    d = q.shape[1]
    rows = n_heads_kv * capacity
    k = decode_via_descriptor(desc, k_raw, rows * d)
    v = decode_via_descriptor(desc, v_raw, rows * d)
    return attention_gen(q, k, v, n_heads_kv, cache_seq_len, capacity, head_major=head_major,
                         scores=scores, scores_stride=scores_stride, impl="scalar", softcap=softcap, kv_index=kv_index)
