"""Pins the CPU oracle's decode / prefill attention against the reference's own test vectors
and closed forms (no GPU)."""
import numpy as np
import pytest

import oracle as O
import textbook as T


def test_lcg_gen_data_matches_hand_computation():
    # engine/src/backend/cpu/x86.rs:1546-1554, evaluated with python ints.
    s, want = 42, []
    for _ in range(64):
        s = (s * 1103515245 + 12345) & 0xFFFFFFFF
        v = (s >> 16) & 0xFFFF
        v = v - 65536 if v >= 32768 else v
        want.append(v / 32768.0)
    assert np.array_equal(O.gen_data(64, 42), np.array(want, np.float32))


def _f16(x):
    return O.f32_to_f16_bits(x).view(np.float16)


@pytest.mark.parametrize("kv", ["f32", "f16"])
def test_avx2_vs_scalar_reference_unit_case(kv):
    # engine/src/backend/cpu/x86.rs:1811-1973: Hq4 Hkv2 d64 L16 cap32, seeds 42/137/53,
    # tolerance 1e-4 (F32) / 1e-3 (F16).
    hq, hkv, d, L, cap = 4, 2, 64, 16, 32
    q = O.gen_data(hq * d, 42).reshape(hq, d)
    k = O.gen_data(hkv * cap * d, 137).reshape(hkv, cap, d)
    v = O.gen_data(hkv * cap * d, 53).reshape(hkv, cap, d)
    if kv == "f16":
        k, v = _f16(k), _f16(v)
    a = O.attention_gen(q, k, v, hkv, L, cap, impl="scalar")
    b = O.attention_gen(q, k, v, hkv, L, cap, impl="avx2")
    tol = 1e-4 if kv == "f32" else 1e-3
    assert np.abs(a - b).max() < tol
    ref, _ = T.decode_attention(q, k, v, hkv, L)
    assert np.abs(a - ref).max() < 1e-5
    assert np.abs(b - ref).max() < 1e-5


def test_f16_conversion_is_rne_like_numpy():
    x = np.concatenate([O.gen_data(4096, 7) * 100.0, [65504.0, 1e-8, -0.0, 6.1e-5]]).astype(np.float32)
    assert np.array_equal(O.f32_to_f16_bits(x), x.astype(np.float16).view(np.uint16))


# engine/tests/test_attention_flash_decoding.rs:260-651 shape matrix (GQA 1/2/4/6, chunk
# boundaries 1023/1024/1025/2047/2500/4096), NMSE < 1e-4 vs the 3-pass reference fed the same
# F16-rounded KV.
@pytest.mark.parametrize("hq,hkv,d,L", [
    (4, 4, 64, 32), (4, 2, 64, 256), (8, 2, 64, 1023), (8, 2, 64, 1024), (8, 2, 64, 1025),
    (12, 2, 128, 2047), (12, 2, 128, 2500), (8, 2, 128, 4096), (14, 2, 64, 1024), (8, 4, 256, 512),
])
@pytest.mark.parametrize("impl", ["scalar", "avx2"])
def test_decode_matrix_vs_f64_textbook(hq, hkv, d, L, impl):
    cap = L + 17
    q = O.gen_data(hq * d, 0x100 + L).reshape(hq, d)
    k = _f16(O.gen_data(hkv * cap * d, 0x200 + L).reshape(hkv, cap, d))
    v = _f16(O.gen_data(hkv * cap * d, 0x300 + L).reshape(hkv, cap, d))
    out, sc = O.attention_gen(q, k, v, hkv, L, cap, scores=True, scores_stride=cap, impl=impl)
    ref, p = T.decode_attention(q, k, v, hkv, L)
    assert T.nmse(out, ref) < 1e-8
    assert np.abs(out - ref).max() < 2e-5
    # scores_out rows sum to 1 (test_attention_flash_decoding.rs:624) and sit at stride `cap`.
    assert np.abs(sc[:, :L].sum(axis=1) - 1.0).max() < 1e-3
    assert np.abs(sc[:, :L] - p).max() < 1e-6
    assert np.all(sc[:, L:] == 0.0)


def test_decode_seq_major_layout_equals_head_major():
    hq, hkv, d, L = 8, 2, 64, 100
    q = O.gen_data(hq * d, 1).reshape(hq, d)
    k = _f16(O.gen_data(hkv * L * d, 2).reshape(hkv, L, d))
    v = _f16(O.gen_data(hkv * L * d, 3).reshape(hkv, L, d))
    ks = np.ascontiguousarray(k.transpose(1, 0, 2))
    vs = np.ascontiguousarray(v.transpose(1, 0, 2))
    a = O.attention_gen(q, k, v, hkv, L, L, head_major=True)
    b = O.attention_gen(q, ks, vs, hkv, L, 0, head_major=False)
    assert np.array_equal(a, b)


def test_decode_closed_form_zero_keys_uniform():
    # engine/src/kv/standard_format.rs:3095-3199: K = 0 => uniform softmax; out = mean of V rows,
    # scores 0.5 / 0.5 for two tokens.
    hq, hkv, d, L = 2, 1, 64, 2
    q = O.gen_data(hq * d, 5).reshape(hq, d)
    k = np.zeros((hkv, 4, d), np.float16)
    v = np.zeros((hkv, 4, d), np.float16)
    v[0, 0], v[0, 1] = 1.0, 3.0
    for impl in ("scalar", "avx2"):
        out, sc = O.attention_gen(q, k, v, hkv, L, 4, scores=True, impl=impl)
        assert np.allclose(out, 2.0, atol=1e-6)
        assert np.allclose(sc, 0.5, atol=1e-7)
    out1 = O.attention_gen(q, k, v, hkv, 1, 4)
    assert np.array_equal(out1, np.ones((hq, d), np.float32))


def test_decode_scalar_nan_and_inf_guards():
    # engine/src/backend/cpu/common.rs:555-584: NaN logit -> -inf; all -inf -> uniform.
    hq, hkv, d, L = 2, 1, 64, 8
    q = O.gen_data(hq * d, 9).reshape(hq, d)
    k = O.gen_data(hkv * L * d, 10).reshape(hkv, L, d)
    v = O.gen_data(hkv * L * d, 11).reshape(hkv, L, d)
    k_nan = k.copy()
    k_nan[0, 3, 0] = np.nan
    out, sc = O.attention_gen(q, k_nan, v, hkv, L, L, scores=True)
    assert np.all(np.isfinite(out)) and np.all(sc[:, 3] == 0.0)
    keep = [0, 1, 2, 4, 5, 6, 7]
    ref, _ = T.decode_attention(q, k[:, keep], v[:, keep], hkv, 7)
    assert np.abs(out - ref).max() < 1e-5
    k_all = np.full_like(k, np.nan)
    out, sc = O.attention_gen(q, k_all, v, hkv, L, L, scores=True)
    assert np.allclose(sc, 1.0 / L)
    assert np.allclose(out, v[0].mean(axis=0), atol=1e-6)


def test_decode_softcap_and_index_extensions():
    # soft-cap definition: engine/kernels/flash_attn_f32_f16.cl:563-565 (after *scale).
    hq, hkv, d, L, cap = 8, 4, 64, 300, 512
    q = O.gen_data(hq * d, 21).reshape(hq, d) * 8.0
    k = _f16(O.gen_data(hkv * cap * d, 22).reshape(hkv, cap, d))
    v = _f16(O.gen_data(hkv * cap * d, 23).reshape(hkv, cap, d))
    out, sc = O.attention_gen(q, k, v, hkv, L, cap, scores=True, softcap=5.0)
    ref, p = T.decode_attention(q, k, v, hkv, L, softcap=5.0)
    assert np.abs(out - ref).max() < 2e-5 and np.abs(sc - p).max() < 1e-6
    # cap -> infinity is the identity
    a = O.attention_gen(q, k, v, hkv, L, cap, softcap=1e9)
    b = O.attention_gen(q, k, v, hkv, L, cap)
    assert np.abs(a - b).max() < 1e-5
    # index list: attention over slots idx[] equals attention over the gathered rows, and the
    # identity index is bit-identical to the plain call (format/selective_read.rs:23-26).
    rng = np.random.default_rng(3)
    idx = np.sort(rng.choice(cap, L, replace=False)).astype(np.int32)
    a = O.attention_gen(q, k, v, hkv, L, cap, kv_index=idx)
    b = O.attention_gen(q, np.ascontiguousarray(k[:, idx]), np.ascontiguousarray(v[:, idx]), hkv, L, L)
    assert np.array_equal(a, b)
    c = O.attention_gen(q, k, v, hkv, L, cap, kv_index=np.arange(L, dtype=np.int32))
    assert np.array_equal(c, O.attention_gen(q, k, v, hkv, L, cap))


# engine/tests/test_prefill_flash_attention.rs:240-559 run_prefill_case matrix
# (q_len, Hq, Hkv, d, q_start_pos, window, seed), NMSE < 1e-4 (1e-5 scalar small).
PREFILL_CASES = [
    (32, 4, 2, 64, 0, 0, 0x10), (64, 4, 2, 64, 0, 0, 0x11), (127, 4, 2, 64, 0, 0, 0x12),
    (128, 4, 2, 64, 0, 0, 0x20), (129, 4, 2, 64, 0, 0, 0x21), (256, 8, 2, 64, 0, 0, 0x22),
    (193, 4, 2, 64, 0, 0, 0x31), (205, 4, 2, 64, 0, 0, 0x32), (200, 12, 2, 128, 0, 0, 0x33),
    (256, 4, 4, 64, 0, 0, 0x40), (256, 12, 2, 128, 0, 0, 0x43), (256, 32, 4, 64, 0, 0, 0x44),
    (512, 4, 2, 64, 0, 64, 0x50), (256, 4, 2, 64, 0, 1024, 0x51), (256, 4, 2, 64, 16, 0, 0x60),
]


@pytest.mark.parametrize("q_len,hq,hkv,d,qsp,window,seed", PREFILL_CASES)
def test_prefill_matrix_vs_f64_textbook(q_len, hq, hkv, d, qsp, window, seed):
    kv_len = qsp + q_len
    cap = max(kv_len, 1)
    q = O.gen_data(q_len * hq * d, seed + 1)
    k = O.gen_data(hkv * cap * d, seed + 2)
    v = O.gen_data(hkv * cap * d, seed + 3)
    out = O.flash_attention_forward_strided(q, k, v, hq, hkv, q_len, kv_len, d, hq * d, d, d, hq * d,
                                            cap * d, qsp, 32, 32, window)
    ref = T.prefill_attention(q.reshape(q_len, hq, d), k.reshape(hkv, cap, d), v.reshape(hkv, cap, d),
                              hkv, kv_len, qsp, window)
    assert T.nmse(out, ref) < 1e-10


def test_prefill_closed_forms():
    # engine/src/kv/standard_format.rs:3095-3199: K=0, V[p]=p => out[r] = r/2.
    s, hq, hkv, d = 64, 2, 1, 64
    q = O.gen_data(s * hq * d, 1).reshape(1, s, hq, d)
    k = np.zeros((1, hkv, s, d), np.float16)
    v = np.broadcast_to(np.arange(s, dtype=np.float16)[None, None, :, None], (1, hkv, s, d)).copy()
    out = O.prefill_attention(q, k, v, hkv, s, s)
    want = (np.arange(s) / 2.0)[None, :, None, None]
    assert np.abs(out - want).max() < 1e-4
    # engine/src/layers/attention.rs:373-710 KATs: single token => out == V row.
    q1 = O.gen_data(hq * d, 2).reshape(1, 1, hq, d)
    k1 = _f16(O.gen_data(hkv * d, 3)).reshape(1, hkv, 1, d)
    v1 = _f16(O.gen_data(hkv * d, 4)).reshape(1, hkv, 1, d)
    o1 = O.prefill_attention(q1, k1, v1, hkv, 1, 1)
    assert np.array_equal(o1[0, 0, 0], v1[0, 0, 0].astype(np.float32))


def test_prefill_wrapper_batch_capacity_and_q_start():
    # standard_format.rs:1262-1310: per-batch strides with capacity > cache_seq_len and
    # q_start_pos = cache_seq_len - seq_len.
    b, s, hq, hkv, d, cap, csl = 2, 40, 4, 2, 64, 96, 70
    q = O.gen_data(b * s * hq * d, 1).reshape(b, s, hq, d)
    k = _f16(O.gen_data(b * hkv * cap * d, 2).reshape(b, hkv, cap, d))
    v = _f16(O.gen_data(b * hkv * cap * d, 3).reshape(b, hkv, cap, d))
    out = O.prefill_attention(q, k, v, hkv, csl, cap)
    for i in range(b):
        ref = T.prefill_attention(q[i], k[i], v[i], hkv, csl, csl - s)
        assert T.nmse(out[i], ref) < 1e-10
