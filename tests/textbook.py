"""Independent f64 / numpy definitions used to pin the CPU oracle and the HIP path.

These are the textbook forms the reference's own tests use as their oracle
(engine/tests/test_attention_flash_decoding.rs:91-160 `reference_attention_f32`,
engine/tests/test_prefill_flash_attention.rs:50-148 `reference_prefill_attention`,
engine/src/bin/test_cuda_quant_attn_device.rs:67-96 host-f64 `ref_attn`), written
in numpy float64 so a dropped term, wrong index or transposed operand in the C
oracle or in a kernel shows up as a large error.
"""
import numpy as np


def nmse(a, b):
    """engine/tests/test_prefill_flash_attention.rs:150-164."""
    a = np.asarray(a, np.float64).ravel()
    b = np.asarray(b, np.float64).ravel()
    num = float(((a - b) ** 2).sum())
    den = float((b ** 2).sum())
    return num if den == 0.0 else num / den


def softmax_rows(s):
    m = s.max(axis=-1, keepdims=True)
    e = np.exp(s - m)
    return e / e.sum(axis=-1, keepdims=True)


def decode_attention(q, k, v, n_heads_kv, cache_seq_len, softcap=0.0, scale=None):
    """q [Hq, d]; k, v HeadMajor [Hkv, cap, d] (any float dtype).  Returns (out, probs) f64."""
    q = np.asarray(q, np.float64)
    hq, d = q.shape
    g = hq // n_heads_kv
    scale = 1.0 / np.sqrt(d) if scale is None else scale
    out = np.zeros((hq, d))
    probs = np.zeros((hq, cache_seq_len))
    for h in range(hq):
        kk = np.asarray(k[h // g, :cache_seq_len], np.float64)
        vv = np.asarray(v[h // g, :cache_seq_len], np.float64)
        s = kk @ q[h] * scale
        if softcap > 0.0:
            s = softcap * np.tanh(s / softcap)
        p = softmax_rows(s[None])[0]
        probs[h] = p
        out[h] = p @ vv
    return out, probs


def prefill_attention(q, k, v, n_heads_kv, kv_len, q_start_pos=0, window=0):
    """q [S, Hq, d]; k, v HeadMajor [Hkv, cap, d].  Causal (+window); masked rows -> 0."""
    q = np.asarray(q, np.float64)
    s_len, hq, d = q.shape
    g = hq // n_heads_kv
    scale = 1.0 / np.sqrt(d)
    out = np.zeros((s_len, hq, d))
    r = np.arange(s_len)[:, None] + q_start_pos
    c = np.arange(kv_len)[None, :]
    ok = c <= r
    if window:
        ok &= (c + window) > r
    for h in range(hq):
        kk = np.asarray(k[h // g, :kv_len], np.float64)
        vv = np.asarray(v[h // g, :kv_len], np.float64)
        s = (q[:, h, :] @ kk.T) * scale
        s = np.where(ok, s, -np.inf)
        m = s.max(axis=1, keepdims=True)
        valid = np.isfinite(m[:, 0])
        m = np.where(np.isfinite(m), m, 0.0)
        e = np.where(ok, np.exp(s - m), 0.0)
        l = e.sum(axis=1, keepdims=True)
        p = np.where(l > 0, e / np.where(l > 0, l, 1.0), 0.0)
        o = p @ vv
        o[~valid] = 0.0
        out[:, h, :] = o
    return out


def round_half_away(x32):
    """Rust f32::round on float32 inputs, exact (done in f64)."""
    x = np.asarray(x32, np.float32).astype(np.float64)
    return np.trunc(x + np.copysign(0.5, x)).astype(np.float32)


def kivi_quantize_block(src, bits):
    """Independent numpy-float32 restatement of BlockQ2_0 / BlockKVQ4 / BlockKVQ8::quantize
    (crates/argus-kv-codec/src/lib.rs:36-59, 125-145, 175-192).  Returns block bytes."""
    src = np.asarray(src, np.float32)
    hi = np.float32((1 << bits) - 1)
    mn = np.float32(src.min())
    mx = np.float32(src.max())
    d = np.float32(np.float32(mx - mn) / hi)
    inv = np.float32(0.0) if d == 0 else np.float32(np.float32(1.0) / d)
    qf = round_half_away(((src - mn).astype(np.float32) * inv).astype(np.float32))
    codes = np.clip(qf, 0.0, hi).astype(np.uint8)
    hdr = np.array([d, mn], np.float32).astype(np.float16).view(np.uint8)
    if bits == 8:
        qs = codes
    elif bits == 4:
        qs = (codes[0::2] | (codes[1::2] << 4)).astype(np.uint8)
    else:
        c = codes.reshape(8, 4)
        qs = (c[:, 0] | (c[:, 1] << 2) | (c[:, 2] << 4) | (c[:, 3] << 6)).astype(np.uint8)
    return np.concatenate([hdr, qs])


def kivi_unpack_codes(blk, bits):
    qs = np.asarray(blk[4:], np.uint8)
    if bits == 8:
        return qs.copy()
    if bits == 4:
        out = np.empty(32, np.uint8)
        out[0::2] = qs & 0x0F
        out[1::2] = qs >> 4
        return out
    out = np.empty(32, np.uint8)
    for j in range(4):
        out[j::4] = (qs >> (2 * j)) & 3
    return out


def kivi_dequantize_block(blk, bits):
    d, m = np.asarray(blk[:4], np.uint8).view(np.float16).astype(np.float32)
    return (kivi_unpack_codes(blk, bits).astype(np.float32) * d + m).astype(np.float32)


def score_reduce(scores, n_kv_heads):
    """scores [n_layers, Hq, L] f64 -> (flat [L], head [Hkv, L]): per layer sum over heads /
    group mean, then MAX over layers (score_reduce.cu:40-56)."""
    scores = np.asarray(scores, np.float64)
    nl, hq, L = scores.shape
    n_rep = hq // n_kv_heads
    flat = scores.sum(axis=1).max(axis=0)
    head = scores.reshape(nl, n_kv_heads, n_rep, L).mean(axis=2).max(axis=0)
    return np.maximum(flat, 0.0), np.maximum(head, 0.0)
