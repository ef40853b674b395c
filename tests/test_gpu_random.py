"""GPU parity on seeded random configurations of every attention entry point: formats, head counts
(GQA groups up to 16), head dims, lengths, window starts, index lists, soft-cap, layouts and batch
sizes drawn together, each checked against the oracle (or, for the prefill, the float64 textbook
attention).  The fixed matrices of the other test files cover the reference's own cases; this file
covers the combinations between them."""
import numpy as np
import pytest

import oracle as O
import textbook as T
from blocks_util import random_blocks
from gpu_util import check_attention_out, check_scores, ctx, dev, host

pytestmark = pytest.mark.gpu

BLOCK_FORMATS = {"q4_0": O.DESC_Q4_0, "q4_1": O.DESC_Q4_1, "q8_0": O.DESC_Q8_0, "q2_0": O.DESC_Q2_0}


# 11332, 11471, 11475: q2_0 rows of three tokens that the matrix-core block kernel put at 2.1-2.2e-3
@pytest.mark.parametrize("case", list(range(60)) + [11332, 11471, 11475])
def test_attention_gen_random(case):
    import argus_hip as A
    rng = np.random.default_rng(7_000_000 + case)
    d = int(rng.choice([64, 128, 256]))
    hkv = int(rng.choice([1, 2, 3, 4, 8]))
    g = int(rng.choice([1, 2, 3, 4, 6, 7, 8, 12, 16][: 7 if d == 256 else 9]))
    hq = hkv * g
    L = int(rng.choice([1, 3, 17, 63, 64, 65, 100, 257, 700, 1500, 4097, 9000]))
    L = min(L, 20_000_000 // (hkv * d))
    cap = L + int(rng.integers(0, 50))
    kind = str(rng.choice(["f16", "f32", "q4_0", "q4_1", "q8_0", "q2_0"]))
    scores = bool(rng.integers(0, 2))
    softcap = float(rng.choice([0.0, 0.0, 7.0, 30.0]))
    use_idx = bool(rng.integers(0, 3) == 0)
    kv_start = 0 if use_idx else int(rng.integers(0, cap - L + 1))
    head_major = bool(rng.integers(0, 4) != 0)
    what = "%s Hq%d Hkv%d d%d L%d cap%d start%d scores%d softcap%g index%d head_major%d" % (
        kind, hq, hkv, d, L, cap, kv_start, scores, softcap, use_idx, head_major)
    q = rng.standard_normal((hq, d)).astype(np.float32) * np.float32(2.0 if softcap else 1.0)
    idx = rng.choice(cap, L, replace=False).astype(np.int32) if use_idx else None
    out = dev(np.zeros((hq, d), np.float32))
    sc = dev(np.zeros((hq, L), np.float32)) if scores else None
    kw = dict(layout=A.HEAD_MAJOR if head_major else A.SEQ_MAJOR, scores=sc, score_stride=L if scores else 0,
              kv_start=kv_start, softcap=softcap, kv_index=dev(idx) if use_idx else None)
    if kind in BLOCK_FORMATS:
        desc = BLOCK_FORMATS[kind]
        kr = random_blocks(desc, hkv * cap * d // 32, case + 1)
        vr = random_blocks(desc, hkv * cap * d // 32, case + 2)
        ctx().attention_gen(dev(q), dev(kr), dev(vr), out, hkv, L, cap, kv_dtype=getattr(A, kind.upper()), **kw)
        kf = O.decode_via_descriptor(desc, kr, hkv * cap * d)
        vf = O.decode_via_descriptor(desc, vr, hkv * cap * d)
    else:
        kf = rng.standard_normal(hkv * cap * d).astype(np.float32)
        vf = rng.standard_normal(hkv * cap * d).astype(np.float32)
        kd, vd = (kf.astype(np.float16), vf.astype(np.float16)) if kind == "f16" else (kf, vf)
        kf, vf = kd.astype(np.float32), vd.astype(np.float32)
        ctx().attention_gen(dev(q), dev(kd), dev(vd), out, hkv, L, cap, **kw)
    shape = (hkv, cap, d) if head_major else (cap, hkv, d)
    kf, vf = kf.reshape(shape), vf.reshape(shape)
    if kv_start:  # a window that starts at kv_start is the same cache with its first rows cut off
        cut = (slice(None), slice(kv_start, None)) if head_major else (slice(kv_start, None),)
        kf, vf = np.ascontiguousarray(kf[cut]), np.ascontiguousarray(vf[cut])
    ref = O.attention_gen(q, kf, vf, hkv, L, cap - kv_start, head_major=head_major, scores=scores, softcap=softcap, kv_index=idx)
    if scores:
        check_attention_out(host(out), ref[0], what)
        check_scores(host(sc), ref[1], what)
    else:
        check_attention_out(host(out), ref, what)


@pytest.mark.parametrize("case", range(40))
def test_kivi_attention_random(case):
    from test_gpu_kivi import run_kivi
    rng = np.random.default_rng(8_000_000 + case)
    bits = int(rng.choice([2, 4, 8]))
    d = int(rng.choice([64, 128, 256]))
    hkv = int(rng.choice([1, 2, 4, 8]))
    hq = hkv * int(rng.choice([1, 2, 4, 7, 8, 12, 16]))
    res_cap = int(rng.choice([32, 64, 128]))
    n = int(rng.choice([1, 5, 31, 32, 33, 100, 129, 300, 1000, 3000]))
    n = min(n, 6_000_000 // (hkv * d))
    res_f16 = bool(rng.integers(0, 2))
    what = "Q%d Hq%d Hkv%d d%d res_cap%d tokens%d res_f16 %d" % (bits, hq, hkv, d, res_cap, n, res_f16)
    k = rng.standard_normal((n, hkv, d)).astype(np.float32)
    v = rng.standard_normal((n, hkv, d)).astype(np.float32)
    q = rng.standard_normal((hq, d)).astype(np.float32)
    c = O.kivi_build(k, v, res_cap, bits)
    scale = 1.0 / np.sqrt(d)
    cr = c
    if res_f16:  # the oracle is fed the f16-rounded residual
        cr = dict(c, res_k=c["res_k"].astype(np.float16).astype(np.float32), res_v=c["res_v"].astype(np.float16).astype(np.float32))
    ref, p = O.kivi_attention(q, cr, scale, scores=True)
    out, sc = run_kivi(q, c, scale, scores="dev", res_f16=res_f16)
    check_attention_out(out, ref, what)
    check_scores(sc, p, what)
    # the same call without scores (what a decode step without an eviction policy issues)
    plain = run_kivi(q, c, scale, res_f16=res_f16)
    plain = plain[0] if isinstance(plain, tuple) else plain
    check_attention_out(plain, ref, what + " (no scores)")


# the cases past 40 are F32-cache draws: in the first six one key dominates a row with |v| near 4 (they
# fail the 2e-3 bar when V is rounded to f16 without its remainder); 31135 is an all-F32 call at
# head_dim 256 with 31 keys, where the roundings of Q, K and the probabilities came to 2.06e-3
# together before the query's low half entered the logits
@pytest.mark.parametrize("case", list(range(40)) + [1428, 2005, 2925, 3625, 3862, 3950, 31135])
def test_prefill_random(case):
    from test_gpu_prefill import f16, run_prefill
    rng = np.random.default_rng(9_000_000 + case)
    d = int(rng.choice([64, 128, 256]))
    hkv = int(rng.choice([1, 2, 4, 8]))
    hq = hkv * int(rng.choice([1, 2, 3, 4, 6, 7, 8, 12, 16]))
    s = int(rng.choice([1, 2, 31, 32, 33, 64, 100, 128, 129, 255, 300, 512, 700, 1024]))
    qsp = int(rng.choice([0, 0, 1, 17, 64, 200, 1000]))
    b = int(rng.choice([1, 1, 2, 3]))
    s = max(1, min(s, 4_000_000 // (b * hq * d)))
    window = int(rng.choice([0, 0, 0, 16, 64, 300]))
    kv_f16, q_f16 = bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
    kv_len = qsp + s
    cap = kv_len + int(rng.integers(0, 40))
    what = "B%d S%d Hq%d Hkv%d d%d q_start%d window%d kv_f16 %d q_f16 %d cap%d" % (b, s, hq, hkv, d, qsp, window, kv_f16, q_f16, cap)
    q = rng.standard_normal((b, s, hq, d)).astype(np.float32)
    k = rng.standard_normal((b, hkv, cap, d)).astype(np.float32)
    v = rng.standard_normal((b, hkv, cap, d)).astype(np.float32)
    if kv_f16:
        k, v = f16(k), f16(v)
    qin = f16(q) if q_f16 else q
    rc, got = run_prefill(qin, k, v, hkv, kv_len, cap, window=window)
    assert rc == 1, what
    for i in range(b):
        r64 = T.prefill_attention(qin[i].astype(np.float32), k[i].astype(np.float32), v[i].astype(np.float32), hkv, kv_len, qsp, window)
        if q_f16:  # the output is rounded to f16 as well: one more 2^-11 relative on values up to ~4
            err = np.abs(got[i].astype(np.float64) - r64)
            assert err.max() <= 4e-3 and err.mean() <= 1e-3, "%s seq %d: max %g mean %g" % (what, i, err.max(), err.mean())
        else:
            check_attention_out(got[i], r64, "%s seq %d" % (what, i))


@pytest.mark.parametrize("case", range(40))
def test_prefill_attention_scores_random(case):
    from test_gpu_pfa import close, run_dev
    rng = np.random.default_rng(10_000_000 + case)
    d = int(rng.choice([8, 24, 64, 128, 192, 256]))
    nkv = int(rng.choice([1, 2, 4, 8]))
    nq = nkv * int(rng.choice([1, 2, 4, 7]))
    seq_len = int(rng.choice([1, 3, 16, 40, 64, 130]))
    q_start = int(rng.choice([0, 0, 5, 100, 700]))
    prefix = q_start + seq_len
    q_window = int(rng.choice([1, 4, 32, 64, 200]))
    window = [None, None, 4, 50][int(rng.integers(0, 4))]
    k_f16, seq_major, per_head = bool(rng.integers(0, 2)), bool(rng.integers(0, 3) == 0), bool(rng.integers(0, 2))
    cap = prefix + int(rng.integers(0, 9))
    q = rng.standard_normal((seq_len, nq, d)).astype(np.float32)
    if seq_major:
        k, kps, khs = rng.standard_normal((cap, nkv, d)).astype(np.float32), nkv * d, d
    else:
        k, kps, khs = rng.standard_normal((nkv, cap, d)).astype(np.float32), d, cap * d
    k_ref = k.astype(np.float16).astype(np.float32) if k_f16 else k
    qw = min(q_window, seq_len)
    init = rng.random((nq, prefix)).astype(np.float32)
    ref_s = init.copy()
    shape = (qw, nq, prefix) if per_head else (qw, prefix)
    ref_p = np.zeros(shape, np.float32)
    O.prefill_attention_scores(q, k_ref.reshape(-1), nq, nkv, d, seq_len, prefix, kps, khs, q_start, q_window, window,
                               sum_out=ref_s, per_row=ref_p, per_head=per_head)
    got_s, got_p = run_dev(q, k.reshape(-1), nq, nkv, d, seq_len, prefix, kps, khs, q_start, q_window, window, True, shape,
                           per_head, k_f16=k_f16, sum_init=init)
    close(got_s, ref_s)
    close(got_p, ref_p)


@pytest.mark.parametrize("case", range(30))
def test_kv_scatter_random(case):
    # Backend::kv_scatter_f32_to_f16[_batch] / kv_scatter_f32_batch (engine/src/backend.rs:425-593):
    # rows [seq, kv_heads, head_dim] F32 into a HeadMajor cache at write_pos, bit for bit (the F16
    # conversion is round-to-nearest-even), everything else untouched.
    from gpu_util import ctx
    rng = np.random.default_rng(12_000_000 + case)
    hkv = int(rng.choice([1, 2, 3, 4, 8, 16]))
    d = int(rng.choice([4, 32, 64, 80, 128, 256]))
    cap = int(rng.choice([1, 7, 64, 129, 1000]))
    seq = int(rng.integers(0, cap + 1))
    pos = int(rng.integers(0, cap - seq + 1))
    to_f16 = bool(rng.integers(0, 2))
    ks = (rng.standard_normal((seq, hkv, d)) * float(rng.choice([1e-6, 1.0, 300.0, 1e5]))).astype(np.float32)
    vs = (rng.standard_normal((seq, hkv, d)) * 3).astype(np.float32)
    dt = np.float16 if to_f16 else np.float32
    kd = rng.standard_normal((hkv, cap, d)).astype(dt)
    vd = rng.standard_normal((hkv, cap, d)).astype(dt)
    dk, dv = dev(kd), dev(vd)
    what = "Hkv%d d%d cap%d seq%d pos%d f16 %d" % (hkv, d, cap, seq, pos, to_f16)
    ctx().kv_scatter(dev(ks) if seq else dk, dev(vs) if seq else dv, dk, dv, hkv, d, cap, pos, seq_len=seq)
    O.kv_scatter(ks, vs, kd, vd, pos)
    view = np.uint16 if to_f16 else np.uint32
    assert np.array_equal(host(dk).view(view), kd.view(view)), what
    assert np.array_equal(host(dv).view(view), vd.view(view)), what


@pytest.mark.parametrize("case", range(30))
def test_score_reduce_random(case):
    # GpuScoreAccumulator's reduce kernels (engine/src/backend/cuda_pc/kernels.cu:305-360 and the
    # per-layer form) against the restated CPU loops: decay, head mean, per-KV-head maximum over the
    # group, maximum over layers; positions past cache_seq_len untouched.
    from gpu_util import ctx
    rng = np.random.default_rng(13_000_000 + case)
    nl = int(rng.choice([1, 2, 5, 28, 33]))
    hkv = int(rng.choice([1, 2, 4, 8, 16]))
    hq = hkv * int(rng.choice([1, 2, 4, 7]))
    L = int(rng.choice([1, 63, 64, 65, 300, 1025, 4000]))
    stride = L + int(rng.integers(0, 70))
    decay = float(rng.choice([0.0, 0.5, 0.9, 1.0]))
    sc = rng.random((nl, hq, stride), dtype=np.float32)
    imp0 = rng.random(stride, dtype=np.float32)
    himp0 = rng.random(hkv * stride, dtype=np.float32)
    lf0 = rng.random(nl * stride, dtype=np.float32)
    imp, himp, lf = imp0.copy(), himp0.copy(), lf0.copy()
    O.score_fused_reduce(sc, imp, himp, decay, nl, hq, hkv, L, stride, stride)
    O.score_reduce_per_layer(sc, lf, decay, nl, hq, L, stride, stride)
    s, di, dh, dl = dev(sc), dev(imp0), dev(himp0), dev(lf0)
    ctx().score_reduce(s, di, dh, decay, nl, hq, hkv, L, stride, stride)
    ctx().score_reduce_per_layer(s, dl, decay, nl, hq, hkv, L, stride, stride)
    what = "layers%d Hq%d Hkv%d L%d stride%d decay%g" % (nl, hq, hkv, L, stride, decay)
    assert np.allclose(host(di), imp, rtol=1e-5, atol=1e-7), what
    assert np.allclose(host(dh), himp, rtol=1e-5, atol=1e-7), what
    assert np.allclose(host(dl), lf, rtol=1e-5, atol=1e-7), what
    assert np.array_equal(host(di)[L:], imp0[L:]), what
