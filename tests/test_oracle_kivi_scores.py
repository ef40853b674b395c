"""Pins the CPU oracle's KIVI codec / container / fused attention, the score policy and the
keep-list compiler against the reference's known-answer vectors (no GPU)."""
import numpy as np
import pytest

import oracle as O
import textbook as T


def _blk(d, m, qs):
    return np.concatenate([np.array([d, m], np.float32).astype(np.float16).view(np.uint8),
                           np.asarray(qs, np.uint8)])


def test_codec_known_answer_blocks():
    # crates/argus-kv-codec/src/lib.rs:303-319: Q2 d=2 m=-1 qs=0b11100100 -> [-1,1,3,5] repeating.
    out = O.kivi_dequantize_block(_blk(2.0, -1.0, [0b11100100] * 8), 2)
    assert np.array_equal(out, np.tile(np.array([-1, 1, 3, 5], np.float32), 8))
    # :382-395: Q4 d=1 m=-2 qs=0x31 -> lo -1, hi +1.
    out = O.kivi_dequantize_block(_blk(1.0, -2.0, [0x31] * 16), 4)
    assert np.array_equal(out, np.tile(np.array([-1, 1], np.float32), 16))
    # Q8: code*d + m.
    out = O.kivi_dequantize_block(_blk(0.5, 1.0, np.arange(32)), 8)
    assert np.array_equal(out, np.arange(32, dtype=np.float32) * 0.5 + 1.0)
    # :32,121,171 size asserts.
    assert [O.kivi_block_bytes(b) for b in (2, 4, 8)] == [12, 20, 36]


@pytest.mark.parametrize("bits", [2, 4, 8])
def test_codec_zero_constant_and_manual_pack(bits):
    # :234-258 zeros -> exactly 0; constant -> d == 0, all codes 0, dequant == f16(value).
    z = O.kivi_quantize_block(np.zeros(32), bits)
    assert not z.any() and np.all(O.kivi_dequantize_block(z, bits) == 0.0)
    c = O.kivi_quantize_block(np.full(32, 42.0), bits)
    assert not c[4:].any() and np.all(O.kivi_dequantize_block(c, bits) == 42.0)
    # :280-300 values (i % levels) -> d == 1, m == 0, codes == values, exact round trip.
    levels = 1 << bits
    src = (np.arange(32) % min(levels, 32)).astype(np.float32)
    if bits == 8:
        src = src * 8.0 + (np.arange(32) == 31) * 7.0  # range 0..255 -> d == 1
    b = O.kivi_quantize_block(src, bits)
    assert np.array_equal(T.kivi_unpack_codes(b, bits).astype(np.float32), src)
    assert np.array_equal(O.kivi_dequantize_block(b, bits), src)


@pytest.mark.parametrize("bits", [2, 4, 8])
def test_codec_bit_exact_vs_independent_numpy_restatement(bits):
    rng = np.random.default_rng(100 + bits)
    for i in range(400):
        src = rng.standard_normal(32).astype(np.float32)
        if i % 7 == 0:
            src[rng.integers(32)] *= 10.0        # outlier channel
        if i % 11 == 0:
            src = np.round(src * 4) / 4          # many exact .5 rounding ties
        a = O.kivi_quantize_block(src, bits)
        b = T.kivi_quantize_block(src, bits)
        assert np.array_equal(a, b), (i, src)
        assert np.array_equal(O.kivi_dequantize_block(a, bits), T.kivi_dequantize_block(b, bits))
        # round-trip invariant |x - x^| <= d/2 + f16 error of d and m
        d = float(a[:2].view(np.float16)[0])
        err = np.abs(O.kivi_dequantize_block(a, bits) - src).max()
        assert err <= d * 0.5 + (1 << bits) * d * 2 ** -10 + np.abs(src).max() * 2 ** -10 + 1e-6


@pytest.mark.parametrize("old,new", [(8, 4), (4, 2), (8, 2), (2, 4), (2, 8), (4, 8), (4, 4)])
def test_requant_vs_independent_numpy_composition(old, new):
    # transition_bits between quantised widths (quant_window_cache.rs:1350-1362): dequantise each
    # block, quantise it again.  Against the independent numpy codec, block by block.
    rng = np.random.default_rng(40 + 10 * old + new)
    n = 300
    src = rng.standard_normal((n, 32)).astype(np.float32)
    src[::9, 5] *= 20.0
    src[7] = 3.25                      # constant block: d == 0 survives the transition
    blocks = np.concatenate([O.kivi_quantize_block(src[i], old) for i in range(n)])
    got = O.kivi_requant(blocks, old, new)
    bo, bn = O.kivi_block_bytes(old), O.kivi_block_bytes(new)
    assert got.size == n * bn
    for i in range(n):
        ref = T.kivi_quantize_block(T.kivi_dequantize_block(blocks[i * bo:(i + 1) * bo], old), new)
        assert np.array_equal(got[i * bn:(i + 1) * bn], ref), i
    c = got[7 * bn:8 * bn]
    assert not c[4:].any() and np.all(O.kivi_dequantize_block(c, new) == 3.25)
    if new >= old:  # widening keeps every value to within the f16 rounding of the new scale and minimum
        for i in range(0, n, 17):
            a = O.kivi_dequantize_block(blocks[i * bo:(i + 1) * bo], old)
            b = O.kivi_dequantize_block(got[i * bn:(i + 1) * bn], new)
            d = float(got[i * bn:i * bn + 2].view(np.float16)[0])
            assert np.abs(a - b).max() <= 0.5 * d + (1 << new) * d * 2.0 ** -10 + np.abs(a).max() * 2.0 ** -10 + 1e-6


def test_requant_reference_transition_case():
    # test_kivi_transition_bits_8_to_4_to_2 (quant_window_cache.rs:3325-3389): 64 tokens of
    # make_input_tensor ramps; Q4 stays close to Q8, Q2 loses more than Q4 did.
    kv_heads, d = 2, 64
    ramp = (np.arange(kv_heads * d, dtype=np.float32) * np.float32(0.01)).reshape(kv_heads, d)  # make_input_tensor, :2682-2692
    k = np.stack([np.float32(i * 0.03) + ramp for i in range(65)])
    c8 = O.kivi_build(k, k + 10.0, 32, 8)
    assert c8["q_tokens"] == 64
    v8, _ = O.kivi_assemble_view(c8)
    c4 = dict(c8, qk=O.kivi_requant(c8["qk"], 8, 4), qv=O.kivi_requant(c8["qv"], 8, 4), bits=4)
    v4, _ = O.kivi_assemble_view(c4)
    c2 = dict(c4, qk=O.kivi_requant(c4["qk"], 4, 2), qv=O.kivi_requant(c4["qv"], 4, 2), bits=2)
    v2, _ = O.kivi_assemble_view(c2)
    mse84 = float(np.mean((v8[:64] - v4[:64]) ** 2))
    mse42 = float(np.mean((v4[:64] - v2[:64]) ** 2))
    assert mse84 < 1.0 and mse42 < 5.0 and mse42 > mse84


def test_codec_round_trip_reference_tolerances():
    # :350-366 KVQ4 i*0.1, max_err range/30+0.02; :399-415 KVQ8 (i-16)*0.5, range/510+0.02;
    # :211-231 Q2 range/6+0.01.
    src = np.arange(32, dtype=np.float32) * 0.1
    assert np.abs(O.kivi_dequantize_block(O.kivi_quantize_block(src, 4), 4) - src).max() < 3.1 / 30 + 0.02
    assert np.abs(O.kivi_dequantize_block(O.kivi_quantize_block(src, 2), 2) - src).max() < 3.1 / 6 + 0.01
    s8 = (np.arange(32, dtype=np.float32) - 16) * 0.5
    assert np.abs(O.kivi_dequantize_block(O.kivi_quantize_block(s8, 8), 8) - s8).max() < 15.5 / 510 + 0.02


def test_container_lazy_flush_timing_and_block_order():
    # engine/src/kv/quant_window_cache.rs:2543-2545, 2760-2786: the flush happens when the
    # residual is full AND another token arrives.
    hkv, d, R = 2, 64, 32
    rng = np.random.default_rng(0)
    k = rng.standard_normal((3 * R + 5, hkv, d)).astype(np.float32)
    v = rng.standard_normal((3 * R + 5, hkv, d)).astype(np.float32)
    c = O.kivi_build(k[:R], v[:R], R, 4)
    assert (c["q_tokens"], c["res_tokens"]) == (0, R)
    c = O.kivi_build(k[:R + 1], v[:R + 1], R, 4)
    assert (c["q_tokens"], c["res_tokens"]) == (R, 1)
    c = O.kivi_build(k, v, R, 4)
    assert (c["q_tokens"], c["res_tokens"]) == (3 * R, 5)
    # block order (quant_window_cache.rs:919-946): K flush -> head -> group -> channel holds
    # channel ch of 32 consecutive tokens; V flush -> head -> token -> d/32 blocks.
    bb = 20
    f, h, ch = 1, 1, 17
    blk = c["qk"].reshape(-1, bb)[f * hkv * d + h * d + ch]
    assert np.array_equal(blk, T.kivi_quantize_block(k[f * R:(f + 1) * R, h, ch], 4))
    t, b = 9, 1
    blk = c["qv"].reshape(-1, bb)[f * hkv * R * 2 + h * R * 2 + t * 2 + b]
    assert np.array_equal(blk, T.kivi_quantize_block(v[f * R + t, h, b * 32:(b + 1) * 32], 4))
    # residual holds the unflushed tail, [Hkv, res_cap, d]
    assert np.array_equal(c["res_k"][:, :5], k[3 * R:].transpose(1, 0, 2))
    # assemble_view: quantised tokens first (within quantisation error), residual exact.
    ak, av = O.kivi_assemble_view(c)
    assert np.array_equal(ak[3 * R:], k[3 * R:]) and np.array_equal(av[3 * R:], v[3 * R:])
    assert np.abs(ak[:3 * R] - k[:3 * R]).max() < 0.5 and np.abs(av[:3 * R] - v[:3 * R]).max() < 0.5


def test_container_multi_group_residual():
    # res_cap = 128 => groups_per_flush = 4; K block index = flush*Hkv*gpf*d + h*gpf*d + gif*d + ch
    # (crates/techniques/kivi/src/kivi_attn.cu:256-262).
    hkv, d, R = 2, 32, 128
    rng = np.random.default_rng(1)
    k = rng.standard_normal((2 * R + 1, hkv, d)).astype(np.float32)
    v = rng.standard_normal((2 * R + 1, hkv, d)).astype(np.float32)
    c = O.kivi_build(k, v, R, 8)
    assert (c["q_tokens"], c["res_tokens"]) == (2 * R, 1)
    f, h, gif, ch = 1, 0, 3, 5
    idx = f * hkv * 4 * d + h * 4 * d + gif * d + ch
    blk = c["qk"].reshape(-1, 36)[idx]
    assert np.array_equal(blk, T.kivi_quantize_block(k[f * R + gif * 32:f * R + gif * 32 + 32, h, ch], 8))


@pytest.mark.parametrize("bits", [2, 4, 8])
def test_kivi_attention_equals_textbook_over_dequantised_view(bits):
    hq, hkv, d, R = 8, 2, 64, 64
    rng = np.random.default_rng(bits)
    n = 3 * R + 11
    k = rng.standard_normal((n, hkv, d)).astype(np.float32)
    v = rng.standard_normal((n, hkv, d)).astype(np.float32)
    q = rng.standard_normal((hq, d)).astype(np.float32)
    c = O.kivi_build(k, v, R, bits)
    scale = 1.0 / np.sqrt(d)
    out, sc = O.kivi_attention(q, c, scale, scores=True)
    ak, av = O.kivi_assemble_view(c)
    ref, p = T.decode_attention(q, ak.transpose(1, 0, 2), av.transpose(1, 0, 2), hkv, n)
    assert np.abs(out - ref).max() < 1e-4 and np.abs(sc - p).max() < 1e-5
    # the CPU fallback of quant_window_format.rs:206-247 (dequantised SeqMajor view ->
    # attention_gen) gives the same answer
    fb = O.attention_gen(q, ak, av, hkv, n, 0, head_major=False)
    assert np.abs(fb - out).max() < 1e-4


def test_kivi_attention_device_test_patterns():
    # engine/src/bin/test_cuda_quant_attn_device.rs:43-258 geometry: 2 Q heads, 1 KV head, d 32,
    # res_cap 32; Q fixture :99-104; Test A residual-only (tol 1e-4, weights sum to 1); Test B
    # Q2-only with exactly representable codes d=0.5 m=1.0 (tol 1e-3).
    nhq, nhkv, hd, R = 2, 1, 32, 32
    scale = 1.0 / np.sqrt(hd)
    q = np.array([[0.1 * ((h * 7 + d) % 5) - 0.2 for d in range(hd)] for h in range(nhq)], np.float32)
    r = 20
    kt = np.array([[0.05 * ((t * 3 + d) % 7) - 0.15 for d in range(hd)] for t in range(r)], np.float32)
    vt = np.array([[0.03 * ((t + d * 2) % 9) for d in range(hd)] for t in range(r)], np.float32)
    res_k = np.zeros((nhkv, R, hd), np.float32)
    res_v = np.zeros((nhkv, R, hd), np.float32)
    res_k[0, :r], res_v[0, :r] = kt, vt
    c = dict(qk=np.zeros(12, np.uint8), qv=np.zeros(12, np.uint8), res_k=res_k, res_v=res_v,
             q_tokens=0, res_tokens=r, res_cap=R, bits=2, kv_heads=nhkv, head_dim=hd)
    out, sc = O.kivi_attention(q, c, scale, scores=True)
    ref, p = T.decode_attention(q, kt[None], vt[None], nhkv, r, scale=scale)
    assert np.abs(out - ref).max() < 1e-4 and np.abs(sc - p).max() < 1e-4
    assert np.abs(sc.sum(axis=1) - 1).max() < 1e-4
    # Test B
    code_k = lambda t, ch: (t + ch) % 4
    code_v = lambda t, d: (t * 2 + d) % 4
    pack = lambda codes: _blk(0.5, 1.0, [sum(codes[i * 4 + j] << (2 * j) for j in range(4)) for i in range(8)])
    qk = np.concatenate([pack([code_k(t, ch) for t in range(32)]) for ch in range(hd)])
    qv = np.concatenate([pack([code_v(t, d) for d in range(32)]) for t in range(32)])
    kq = np.array([[code_k(t, ch) * 0.5 + 1.0 for ch in range(hd)] for t in range(32)], np.float32)
    vq = np.array([[code_v(t, d) * 0.5 + 1.0 for d in range(hd)] for t in range(32)], np.float32)
    c = dict(qk=qk, qv=qv, res_k=res_k, res_v=res_v, q_tokens=32, res_tokens=0, res_cap=R, bits=2,
             kv_heads=nhkv, head_dim=hd)
    out = O.kivi_attention(q, c, scale)
    ref, _ = T.decode_attention(q, kq[None], vq[None], nhkv, 32, scale=scale)
    assert np.abs(out - ref).max() < 1e-3


def test_score_producer_known_answers():
    # crates/techniques/attn-score/src/lib.rs:888-953.
    p = O.ScoreProducer(4, 1)
    p.begin_step()
    p.accumulate_layer_gqa(np.array([0.1, 0.2, 0.3, 0.4], np.float32), 4, 4, 1)
    p.accumulate_layer_gqa(np.array([0.4, 0.1, 0.1, 0.4], np.float32), 4, 4, 1)
    p.end_step()
    assert np.allclose(p.importance, [0.4, 0.2, 0.3, 0.4])
    p = O.ScoreProducer(4, 1)
    for _ in range(3):
        p.begin_step()
        p.accumulate_layer_gqa(np.array([1, 2, 3, 4], np.float32), 4, 4, 1)
        p.end_step()
    assert np.array_equal(p.importance, np.array([3, 6, 9, 12], np.float32))
    # one-hot, 4 Q heads / 2 KV heads: head importance 0.5, flat 1.0
    p = O.ScoreProducer(4, 2)
    sc = np.zeros((4, 4), np.float32)
    sc[0, 1] = 1.0
    p.begin_step()
    p.accumulate_layer_gqa(sc, 4, 4, 4)
    p.end_step()
    assert p.importance[1] == 1.0 and p.head_importance[1] == 0.5 and p.head_importance[4 + 1] == 0.0


def test_score_fused_reduce_known_answers():
    # engine/src/bin/test_cuda_gpu_score_device.rs: 2 layers x 2 Q heads x 1 KV head.
    nl, hq, hkv, max_seq, L = 2, 2, 1, 8, 3
    sc = np.zeros((nl, hq, max_seq), np.float32)
    sc[0, 0, :3], sc[0, 1, :3] = [0.1, 0.2, 0.7], [0.3, 0.3, 0.4]
    sc[1, 0, :3], sc[1, 1, :3] = [0.5, 0.4, 0.1], [0.2, 0.2, 0.6]
    imp, himp = np.zeros(max_seq, np.float32), np.zeros(hkv * max_seq, np.float32)
    O.score_fused_reduce(sc, imp, himp, 1.0, nl, hq, hkv, L, max_seq, max_seq)
    assert np.abs(imp[:3] - [0.7, 0.6, 1.1]).max() < 1e-5
    assert np.abs(himp[:3] - [0.35, 0.30, 0.55]).max() < 1e-5
    assert not imp[3:].any()
    imp[:] = 0
    himp[:] = 0
    for _ in range(2):
        O.score_fused_reduce(sc, imp, himp, 0.5, nl, hq, hkv, L, max_seq, max_seq)
    assert np.abs(imp[:3] - 1.5 * np.array([0.7, 0.6, 1.1])).max() < 1e-5
    # per-layer variant: no cross-layer MAX (score_reduce.cu:80-90)
    lf = np.zeros(nl * max_seq, np.float32)
    O.score_reduce_per_layer(sc, lf, 1.0, nl, hq, L, max_seq, max_seq)
    assert np.abs(lf[:3] - [0.4, 0.5, 1.1]).max() < 1e-6 and np.abs(lf[8:11] - [0.7, 0.6, 0.7]).max() < 1e-6
    # CPU producer and fused GPU semantics agree on a single step (decay 0)
    rng = np.random.default_rng(0)
    nl, hq, hkv, L = 3, 8, 4, 50
    s = rng.random((nl, hq, L)).astype(np.float32)
    imp, himp = np.zeros(L, np.float32), np.zeros(hkv * L, np.float32)
    O.score_fused_reduce(s, imp, himp, 1.0, nl, hq, hkv, L, L, L)
    p = O.ScoreProducer(L, hkv)
    p.begin_step()
    for l in range(nl):
        p.accumulate_layer_gqa(s[l], L, L, hq)
    p.end_step()
    assert np.allclose(p.importance, imp, rtol=1e-6) and np.allclose(p.head_importance, himp, rtol=1e-6)
    flat, head = T.score_reduce(s, hkv)
    assert np.allclose(imp, flat, rtol=1e-5) and np.allclose(himp.reshape(hkv, L), head, rtol=1e-5)


def test_keep_list_known_answers():
    # crates/techniques/streaming-llm/src/lib.rs:238-307, sink 4 / window 6.
    assert O.streaming_keep(4, 6, 15, 0).tolist() == [0, 1, 2, 3, 9, 10, 11, 12, 13, 14]
    assert O.streaming_keep(4, 6, 8, 0) is None and O.streaming_keep(4, 6, 10, 0) is None
    assert O.streaming_keep(4, 6, 11, 0).tolist() == [0, 1, 2, 3, 5, 6, 7, 8, 9, 10]
    assert O.streaming_keep(4, 6, 20, 7).tolist() == [0, 1, 2, 3, 17, 18, 19]
    assert O.streaming_keep(4, 6, 20, 2).tolist() == [0, 1, 2, 3, 19]
    # benchmark configuration 5: history 8192, sink 4 + recent 2044 -> {0..3} U {6148..8191}
    k = O.streaming_keep(4, 2044, 8192, 0)
    assert len(k) == 2048 and k[:4].tolist() == [0, 1, 2, 3] and k[4] == 6148 and k[-1] == 8191


def test_keep_top_k_vs_brute_force_stable_selection():
    # crates/argus-extension-api/src/lib.rs:788-810: stable descending sort, ties keep position
    # order; prefix clamp; recent_start = max(current - recent, prefix).
    rng = np.random.default_rng(5)
    for _ in range(200):
        cur = int(rng.integers(1, 60))
        prefix, recent, heavy = (int(rng.integers(0, 12)) for _ in range(3))
        score = rng.integers(0, 4, cur).astype(np.float32)   # many ties
        got = O.compile_keep_top_k(cur, prefix, recent, heavy, score).tolist()
        p = min(prefix, cur)
        rs = max(max(cur - recent, 0), p)
        mid = sorted(range(p, rs), key=lambda i: -score[i])   # python sort is stable
        want = list(range(p)) + sorted(mid[:heavy]) + list(range(rs, cur))
        assert got == want


def test_compaction_and_scatter_vs_naive_model():
    # engine/src/kv/naive_reference.rs:21-120 style [pos][head][d] model.
    rng = np.random.default_rng(2)
    hkv, cap, d = 3, 40, 32
    src = rng.standard_normal((hkv, cap, d)).astype(np.float16)
    keep = np.array([0, 1, 5, 7, 30, 39], np.int32)
    dst = O.compact_keep(src, keep, 16)
    assert np.array_equal(dst[:, :6], src[:, keep]) and not dst[:, 6:].any()
    # kv_scatter (cuda_pc/kernels.cu:305-360): src [S, Hkv, d] f32 -> dst[h, write_pos+s, :] f16 RNE
    s = 5
    ks = rng.standard_normal((s, hkv, d)).astype(np.float32)
    vs = rng.standard_normal((s, hkv, d)).astype(np.float32)
    kd = np.zeros((hkv, cap, d), np.float16)
    vd = np.zeros((hkv, cap, d), np.float16)
    O.kv_scatter(ks, vs, kd, vd, 11)
    assert np.array_equal(kd[:, 11:16], ks.transpose(1, 0, 2).astype(np.float16))
    assert np.array_equal(vd[:, 11:16], vs.transpose(1, 0, 2).astype(np.float16))
    assert not kd[:, :11].any() and not kd[:, 16:].any()


@pytest.mark.parametrize("bits", [2, 4, 8])
def test_f16_view_dequant_flush_and_scatter_match_assembled_view(bits):
    # The F16 attention view built flush by flush (kivi_q2.cu:18-116) must equal the C oracle's
    # dequantised view (an independent walk over the same container) rounded to f16.
    hkv, d, R, n = 3, 64, 64, 64 * 3 + 17
    rng = np.random.default_rng(90 + bits)
    k = rng.standard_normal((n, hkv, d)).astype(np.float32)
    v = rng.standard_normal((n, hkv, d)).astype(np.float32)
    c = O.kivi_build(k, v, R, bits)
    ak, av = O.kivi_assemble_view(c)
    vk = np.full((n + 3, hkv, d), 7.0, np.float16)
    vv = np.full((n + 3, hkv, d), 7.0, np.float16)
    gpf = R // 32
    for f in range(c["q_tokens"] // R):
        O.kivi_dequant_flush_f16(c["qk"], vk, hkv, d, gpf, f * R, f * hkv * gpf * d, bits, True)
        O.kivi_dequant_flush_f16(c["qv"], vv, hkv, d, R, f * R, f * hkv * R * (d // 32), bits, False)
    O.kivi_scatter_residual_f16(c["res_k"], vk, hkv, R, d, c["res_tokens"], c["q_tokens"])
    O.kivi_scatter_residual_f16(c["res_v"], vv, hkv, R, d, c["res_tokens"], c["q_tokens"])
    assert np.array_equal(vk[:n], ak.astype(np.float16)) and np.array_equal(vv[:n], av.astype(np.float16))
    assert (vk[n:] == 7.0).all() and (vv[n:] == 7.0).all()
