"""GPU parity: KIVI fused dequant decode, residual append and on-device quantise-at-flush."""
import ctypes as C

import numpy as np
import pytest

import oracle as O
import textbook as T
from gpu_util import check_attention_out, check_scores, ctx, dev, host, normal

pytestmark = pytest.mark.gpu


def run_kivi(q, c, scale, scores=None, res_f16=False, softcap=0.0):
    """scores: None | 'host' | 'dev'."""
    import torch
    hq, d = q.shape
    total = c["q_tokens"] + c["res_tokens"]
    out = torch.full((hq, d), float("nan"), device="cuda")
    rk, rv = c["res_k"], c["res_v"]
    if res_f16:
        rk, rv = rk.astype(np.float16), rv.astype(np.float16)
    kw = {}
    sh = sd = None
    if scores == "host":
        sh = np.full((hq, total), -3.0, np.float32)
        kw["scores_host"] = sh
    elif scores == "dev":
        sd = torch.full((hq, total + 5), -3.0, device="cuda")
        kw.update(scores_dev=sd, score_stride=total + 5)
    ctx().attention_gen_quant(dev(q), dev(c["qk"]), dev(c["qv"]), dev(rk), dev(rv), out, c["kv_heads"],
                              c["q_tokens"], c["res_tokens"], c["res_cap"], scale, c["bits"],
                              softcap=softcap, **kw)
    o = host(out)
    if scores == "host":
        return o, sh
    if scores == "dev":
        return o, host(sd)[:, :total]
    return o


def _blk(d, m, qs):
    return np.concatenate([np.array([d, m], np.float32).astype(np.float16).view(np.uint8), np.asarray(qs, np.uint8)])


def test_reference_device_test_patterns():
    # engine/src/bin/test_cuda_quant_attn_device.rs:43-258 (Test A residual-only with host score
    # read-back, Test B Q2-only with exactly representable codes), its own tolerances.
    assert all(ctx().has_quant_attn_kernel(b) for b in (2, 4, 8)) and not ctx().has_quant_attn_kernel(3)
    nhq, nhkv, hd, R = 2, 1, 32, 32
    scale = 1.0 / np.sqrt(hd)
    q = np.array([[0.1 * ((h * 7 + d) % 5) - 0.2 for d in range(hd)] for h in range(nhq)], np.float32)
    # head_dim 32 is below the kernels' coverage (64/128/256): the call must decline with a
    # negative code (the engine then uses its dequantised-view fallback), never crash.
    import argus_hip as A
    import torch
    z = torch.zeros(64, device="cuda")
    rc = ctx().attention_gen_quant(dev(q), z, z, z, z, torch.zeros((nhq, hd), device="cuda"), nhkv, 0, 20, R,
                                   scale, 2, check=False)
    assert rc == A.ERR_UNSUPPORTED
    # the same analytic patterns at head_dim 64
    hd = 64
    scale = 1.0 / np.sqrt(hd)
    q = np.array([[0.1 * ((h * 7 + d) % 5) - 0.2 for d in range(hd)] for h in range(nhq)], np.float32)
    r = 20
    kt = np.array([[0.05 * ((t * 3 + d) % 7) - 0.15 for d in range(hd)] for t in range(r)], np.float32)
    vt = np.array([[0.03 * ((t + d * 2) % 9) for d in range(hd)] for t in range(r)], np.float32)
    res_k = np.zeros((nhkv, R, hd), np.float32)
    res_v = np.zeros((nhkv, R, hd), np.float32)
    res_k[0, :r], res_v[0, :r] = kt, vt
    c = dict(qk=np.zeros(12, np.uint8), qv=np.zeros(12, np.uint8), res_k=res_k, res_v=res_v, q_tokens=0,
             res_tokens=r, res_cap=R, bits=2, kv_heads=nhkv, head_dim=hd)
    out, sc = run_kivi(q, c, scale, scores="host")
    ref, p = T.decode_attention(q, kt[None], vt[None], nhkv, r, scale=scale)
    assert np.abs(out - ref).max() < 1e-4 and np.abs(sc - p).max() < 1e-4
    assert np.abs(sc.sum(axis=1) - 1).max() < 1e-4
    code_k = lambda t, ch: (t + ch) % 4
    code_v = lambda t, d: (t * 2 + d) % 4
    pack = lambda codes: _blk(0.5, 1.0, [sum(codes[i * 4 + j] << (2 * j) for j in range(4)) for i in range(8)])
    qk = np.concatenate([pack([code_k(t, ch) for t in range(32)]) for ch in range(hd)])
    qv = np.concatenate([pack([code_v(t, b * 32 + d) for d in range(32)]) for t in range(32) for b in range(hd // 32)])
    kq = np.array([[code_k(t, ch) * 0.5 + 1.0 for ch in range(hd)] for t in range(32)], np.float32)
    vq = np.array([[code_v(t, d) * 0.5 + 1.0 for d in range(hd)] for t in range(32)], np.float32)
    c = dict(qk=qk, qv=qv, res_k=res_k, res_v=res_v, q_tokens=32, res_tokens=0, res_cap=R, bits=2,
             kv_heads=nhkv, head_dim=hd)
    out = run_kivi(q, c, scale)
    ref, _ = T.decode_attention(q, kq[None], vq[None], nhkv, 32, scale=scale)
    assert np.abs(out - ref).max() < 1e-3


@pytest.mark.parametrize("bits", [2, 4, 8])
@pytest.mark.parametrize("hq,hkv,d,R,n", [(8, 2, 64, 64, 203), (4, 4, 128, 32, 97), (8, 4, 256, 128, 300),
                                          (14, 2, 64, 128, 128), (32, 8, 128, 128, 1024),
                                          (16, 8, 256, 128, 2100), (32, 4, 256, 64, 700), (3, 1, 256, 32, 1500),
                                          # GQA groups of 12 and 16: two head tiles per KV head
                                          (24, 2, 128, 64, 500), (32, 2, 64, 32, 300), (16, 1, 256, 128, 260)])
def test_kivi_attention_vs_oracle(bits, hq, hkv, d, R, n):
    rng = np.random.default_rng(bits * 1000 + n)
    k = rng.standard_normal((n, hkv, d)).astype(np.float32)
    v = rng.standard_normal((n, hkv, d)).astype(np.float32)
    q = rng.standard_normal((hq, d)).astype(np.float32)
    c = O.kivi_build(k, v, R, bits)
    scale = 1.0 / np.sqrt(d)
    ref, p = O.kivi_attention(q, c, scale, scores=True)
    out, sc = run_kivi(q, c, scale, scores="dev")
    check_attention_out(out, ref)
    check_scores(sc, p)
    out_h, sc_h = run_kivi(q, c, scale, scores="host")
    assert np.array_equal(out_h, out) and np.array_equal(sc_h, sc)
    # independent: textbook attention over the dequantised view
    ak, av = O.kivi_assemble_view(c)
    r64, _ = T.decode_attention(q, ak.transpose(1, 0, 2), av.transpose(1, 0, 2), hkv, n)
    check_attention_out(out, r64)


@pytest.mark.parametrize("bits", [2, 4, 8])
@pytest.mark.parametrize("hq,hkv,d,R,n", [(8, 4, 256, 128, 900), (32, 8, 128, 128, 700), (14, 2, 64, 32, 333)])
def test_kivi_soft_cap(bits, hq, hkv, d, R, n):
    # The logit soft-cap (cap * tanh(logit / cap)) has no counterpart in the reference's KIVI kernels;
    # it is checked against the float64 textbook attention over the dequantised view, with queries
    # large enough that the cap bites.
    rng = np.random.default_rng(bits * 100 + n)
    k = rng.standard_normal((n, hkv, d)).astype(np.float32)
    v = rng.standard_normal((n, hkv, d)).astype(np.float32)
    q = (3.0 * rng.standard_normal((hq, d))).astype(np.float32)
    c = O.kivi_build(k, v, R, bits)
    scale = 1.0 / np.sqrt(d)
    ak, av = O.kivi_assemble_view(c)
    for cap in (50.0, 4.0):
        out, sc = run_kivi(q, c, scale, scores="dev", softcap=cap)
        r64, p64 = T.decode_attention(q, ak.transpose(1, 0, 2), av.transpose(1, 0, 2), hkv, n, softcap=cap, scale=scale)
        check_attention_out(out, r64, "cap %g" % cap)
        check_scores(sc, p64, "cap %g" % cap)


@pytest.mark.parametrize("bits", [4, 8])
def test_config4_llama8b_kivi(bits):
    # benchmark configuration 4: Hq32 Hkv8 d128, 8192 appended tokens, res_cap 128 -> q_tokens 8064 +
    # residual 128; N(0,1) with 1% outlier channels x10; residual F32 (ABI) and F16 (the benchmark's).
    hq, hkv, d, n, R = 32, 8, 128, 8192, 128
    rng = np.random.default_rng(4)
    k = rng.standard_normal((n, hkv, d), dtype=np.float32)
    v = rng.standard_normal((n, hkv, d), dtype=np.float32)
    for h in range(hkv):
        k[:, h, rng.choice(d, 2, replace=False)] *= 10.0
        v[:, h, rng.choice(d, 2, replace=False)] *= 10.0
    q = rng.standard_normal((hq, d), dtype=np.float32)
    c = O.kivi_build(k, v, R, bits)
    assert (c["q_tokens"], c["res_tokens"]) == (8064, 128)
    scale = 1.0 / np.sqrt(d)
    ref, p = O.kivi_attention(q, c, scale, scores=True)
    out, sc = run_kivi(q, c, scale, scores="dev")
    check_attention_out(out, ref)
    check_scores(sc, p)
    # F16 residual window: compare with the oracle fed the f16-rounded residual
    c16 = dict(c, res_k=c["res_k"].astype(np.float16).astype(np.float32),
               res_v=c["res_v"].astype(np.float16).astype(np.float32))
    ref16 = O.kivi_attention(q, c16, scale)
    out16 = run_kivi(q, c, scale, res_f16=True)
    check_attention_out(out16, ref16)


def test_batched_caches_match_single_calls():
    # several caches (sequences / layers) of one geometry in a single launch == one call each
    import torch
    nb, hq, hkv, d, R, n, bits = 3, 8, 2, 128, 64, 64 * 3 + 9, 4
    rng = np.random.default_rng(77)
    caches = [O.kivi_build(rng.standard_normal((n, hkv, d)).astype(np.float32),
                           rng.standard_normal((n, hkv, d)).astype(np.float32), R, bits) for _ in range(nb)]
    q = rng.standard_normal((nb, hq, d)).astype(np.float32)
    nbytes = caches[0]["qk"].size
    qk = dev(np.stack([c["qk"] for c in caches]))
    qv = dev(np.stack([c["qv"] for c in caches]))
    rk = dev(np.stack([c["res_k"] for c in caches]))
    rv = dev(np.stack([c["res_v"] for c in caches]))
    out = torch.empty((nb, hq, d), device="cuda")
    total = caches[0]["q_tokens"] + caches[0]["res_tokens"]
    sc = torch.zeros((nb, hq, total), device="cuda")
    ctx().attention_gen_quant(dev(q), qk, qv, rk, rv, out, hkv, caches[0]["q_tokens"], caches[0]["res_tokens"], R,
                              1.0 / np.sqrt(d), bits, scores_dev=sc, score_stride=total, batch=nb,
                              block_batch_stride_bytes=nbytes, res_batch_stride=hkv * R * d)
    for i, c in enumerate(caches):
        ref, p = O.kivi_attention(q[i], c, 1.0 / np.sqrt(d), scores=True)
        check_attention_out(host(out)[i], ref, "cache %d" % i)
        check_scores(host(sc)[i], p, "cache %d" % i)


def test_scores_as_logits_and_statistics():
    # the opt-in score form of the decode calls (rows keep their logits, (max, sum) beside them):
    # probabilities rebuilt from it equal the default form's, outputs are identical
    import torch
    nb, hq, hkv, d, R, n, bits = 2, 8, 2, 128, 64, 64 * 5 + 17, 4
    rng = np.random.default_rng(78)
    caches = [O.kivi_build(rng.standard_normal((n, hkv, d)).astype(np.float32),
                           rng.standard_normal((n, hkv, d)).astype(np.float32), R, bits) for _ in range(nb)]
    q = dev(rng.standard_normal((nb, hq, d)).astype(np.float32))
    nbytes = caches[0]["qk"].size
    qk, qv = dev(np.stack([c["qk"] for c in caches])), dev(np.stack([c["qv"] for c in caches]))
    rk, rv = dev(np.stack([c["res_k"] for c in caches])), dev(np.stack([c["res_v"] for c in caches]))
    total = caches[0]["q_tokens"] + caches[0]["res_tokens"]
    outs, scs = [], []
    st = torch.zeros((nb, hq, 2), device="cuda")
    for stats in (None, st):
        out = torch.empty((nb, hq, d), device="cuda")
        sc = torch.zeros((nb, hq, total), device="cuda")
        ctx().attention_gen_quant(q, qk, qv, rk, rv, out, hkv, caches[0]["q_tokens"], caches[0]["res_tokens"], R,
                                  1.0 / np.sqrt(d), bits, scores_dev=sc, score_stride=total, batch=nb,
                                  block_batch_stride_bytes=nbytes, res_batch_stride=hkv * R * d, score_stats=stats)
        outs.append(out)
        scs.append(sc)
    assert torch.equal(outs[0], outs[1])
    assert torch.allclose(torch.exp(scs[1] - st[..., 0:1]) / st[..., 1:2], scs[0], rtol=1e-5, atol=0)
    imp, himp = torch.zeros(total, device="cuda"), torch.zeros(hkv * total, device="cuda")
    imp2, himp2 = torch.zeros(total, device="cuda"), torch.zeros(hkv * total, device="cuda")
    ctx().score_reduce(scs[0], imp, himp, 1.0, nb, hq, hkv, total, total, total)
    ctx().score_reduce(scs[1], imp2, himp2, 1.0, nb, hq, hkv, total, total, total, stats=st)
    assert torch.equal(imp, imp2) and torch.equal(himp, himp2)


def test_gather_update_and_flush_bit_exact():
    # Drive the container on the device: append tokens through gather_update_quant, quantise a
    # full residual with quant_flush, and compare blocks bit for bit with the CPU container
    # (engine/src/kv/quant_window_cache.rs:919-946, 2518-2562).
    import torch
    hkv, d, R = 4, 128, 64
    rng = np.random.default_rng(11)
    n = 2 * R + 7
    k = rng.standard_normal((n, hkv, d)).astype(np.float32)
    v = rng.standard_normal((n, hkv, d)).astype(np.float32)
    k[:, 1, 5] *= 10.0
    k[R:2 * R, 2, 9] = 0.25            # constant channel group -> d == 0
    v[3, 0, :32] = np.round(v[3, 0, :32] * 2) / 2   # rounding ties
    for bits in (2, 4, 8):
        bb = O.kivi_block_bytes(bits)
        c = O.kivi_build(k, v, R, bits)
        res_k = torch.zeros((hkv, R, d), device="cuda")
        res_v = torch.zeros((hkv, R, d), device="cuda")
        nblk = 2 * hkv * R * d // 32
        qk = torch.zeros(nblk * bb, dtype=torch.uint8, device="cuda")
        qv = torch.zeros(nblk * bb, dtype=torch.uint8, device="cuda")
        kd, vd = dev(k), dev(v)
        res_pos, kb, vb = 0, 0, 0
        s = 0
        while s < n:
            if res_pos >= R:
                ctx().quant_flush(res_k, res_v, qk, qv, hkv, R, d, R, kb, vb, bits)
                kb += hkv * (R // 32) * d
                vb += hkv * R * (d // 32)
                res_pos = 0
            step = min(3 if s % 2 else 1, R - res_pos, n - s)   # mix single- and multi-token appends
            ctx().gather_update_quant(kd[s:s + step], res_k, hkv, R, d, step, res_pos)
            ctx().gather_update_quant(vd[s:s + step], res_v, hkv, R, d, step, res_pos)
            res_pos += step
            s += step
        assert res_pos == c["res_tokens"] and kb * 32 // (hkv * d) == c["q_tokens"]
        assert np.array_equal(host(qk)[:kb * bb], c["qk"][:kb * bb]), "K blocks differ (bits %d)" % bits
        assert np.array_equal(host(qv)[:vb * bb], c["qv"][:vb * bb]), "V blocks differ (bits %d)" % bits
        assert np.array_equal(host(res_k)[:, :res_pos], c["res_k"][:, :res_pos])
        # and the device-built cache feeds the fused kernel
        q = rng.standard_normal((8, d)).astype(np.float32)
        out = torch.empty((8, d), device="cuda")
        ctx().attention_gen_quant(dev(q), qk, qv, res_k, res_v, out, hkv, c["q_tokens"], res_pos, R,
                                  1.0 / np.sqrt(d), bits)
        check_attention_out(host(out), O.kivi_attention(q, c, 1.0 / np.sqrt(d)))


def test_flush_bit_exact_on_adversarial_blocks():
    import torch
    hkv, d, R = 1, 64, 32
    rng = np.random.default_rng(5)
    res = np.zeros((hkv, R, d), np.float32)
    res[0] = rng.standard_normal((R, d)).astype(np.float32)
    res[0, :, 0] = 0.0                                   # zeros
    res[0, :, 1] = 42.0                                  # constant
    res[0, :, 2] = np.arange(32) % 4                     # exact levels
    res[0, :, 3] = np.arange(32) * 0.1                   # reference round-trip input
    res[0, :, 4] = -10.0 + np.arange(32) * 9.0 / 31.0    # negative range
    res[0, :, 5] = np.linspace(-1e-3, 1e-3, 32)          # tiny range
    res[0, :, 6] = np.linspace(-6e4, 6e4, 32)            # near f16 max
    res[0, :, 7] = (np.arange(32) % 2) * 7.5             # .5 ties at 4 bits
    c_in = res.transpose(1, 0, 2).copy()                 # [R, hkv, d] tokens
    for bits in (2, 4, 8):
        bb = O.kivi_block_bytes(bits)
        # one more token forces the CPU container to flush
        c = O.kivi_build(np.concatenate([c_in, c_in[:1]]), np.concatenate([c_in, c_in[:1]]), R, bits)
        qk = torch.zeros(hkv * d * bb, dtype=torch.uint8, device="cuda")
        qv = torch.zeros(hkv * R * (d // 32) * bb, dtype=torch.uint8, device="cuda")
        r = dev(res)
        ctx().quant_flush(r, r, qk, qv, hkv, R, d, R, 0, 0, bits)
        assert np.array_equal(host(qk), c["qk"][:qk.numel()])
        assert np.array_equal(host(qv), c["qv"][:qv.numel()])


def test_kivi_argument_errors():
    import torch
    import argus_hip as A
    z = torch.zeros(4096, device="cuda")
    q = torch.zeros((8, 128), device="cuda")
    c = ctx()
    assert c.attention_gen_quant(q, z, z, z, z, q.clone(), 2, 32, 0, 32, 0.1, 3, check=False) == A.ERR_UNSUPPORTED
    assert "bits" in c.last_error()
    assert c.attention_gen_quant(q, z, z, z, z, q.clone(), 3, 32, 0, 32, 0.1, 4, check=False) == A.ERR_INVALID
    assert c.attention_gen_quant(q, z, z, z, z, q.clone(), 2, 0, 0, 32, 0.1, 4, check=False) == A.ERR_INVALID
    assert c.attention_gen_quant(q, z, z, z, z, q.clone(), 2, 33, 0, 32, 0.1, 4, check=False) == A.ERR_INVALID
    assert c.gather_update_quant(z, z, 2, 32, 128, 4, 30, check=False) == A.ERR_INVALID
    assert c.quant_flush(z, z, z, z, 2, 32, 128, 48, 0, 0, 4, check=False) == A.ERR_INVALID


@pytest.mark.parametrize("bits", [2, 4, 8])
@pytest.mark.parametrize("hkv,d,R,n", [(3, 64, 64, 64 * 3 + 17), (8, 128, 128, 128 * 2 + 128), (2, 256, 32, 97)])
def test_f16_view_dequant_flush_and_scatter_bit_exact(bits, hkv, d, R, n):
    # CudaQuantAttnBackend::{dequant_flush, scatter_residual}: the F16 attention view built on the
    # device flush by flush equals the oracle's, bit for bit, and nothing outside the rows is touched.
    import torch
    rng = np.random.default_rng(300 + bits + n)
    k = rng.standard_normal((n, hkv, d)).astype(np.float32)
    v = rng.standard_normal((n, hkv, d)).astype(np.float32)
    k[:, 0, 1] *= 10.0
    c = O.kivi_build(k, v, R, bits)
    gpf = R // 32
    ref_k = np.full((n + 2, hkv, d), 7.0, np.float16)
    ref_v = ref_k.copy()
    dev_k = torch.full((n + 2, hkv, d), 7.0, device="cuda", dtype=torch.float16)
    dev_v = dev_k.clone()
    qk, qv, rk, rv = dev(c["qk"]), dev(c["qv"]), dev(c["res_k"]), dev(c["res_v"])
    for f in range(c["q_tokens"] // R):
        kb, vb = f * hkv * gpf * d, f * hkv * R * (d // 32)
        O.kivi_dequant_flush_f16(c["qk"], ref_k, hkv, d, gpf, f * R, kb, bits, True)
        O.kivi_dequant_flush_f16(c["qv"], ref_v, hkv, d, R, f * R, vb, bits, False)
        ctx().quant_dequant_flush(qk, dev_k, hkv, d, gpf, f * R, kb, bits, True)
        ctx().quant_dequant_flush(qv, dev_v, hkv, d, R, f * R, vb, bits, False)
    O.kivi_scatter_residual_f16(c["res_k"], ref_k, hkv, R, d, c["res_tokens"], c["q_tokens"])
    O.kivi_scatter_residual_f16(c["res_v"], ref_v, hkv, R, d, c["res_tokens"], c["q_tokens"])
    ctx().quant_scatter_residual(rk, dev_k, hkv, R, d, c["res_tokens"], c["q_tokens"])
    ctx().quant_scatter_residual(rv, dev_v, hkv, R, d, c["res_tokens"], c["q_tokens"])
    got_k, got_v = host(dev_k), host(dev_v)
    assert np.array_equal(got_k.view(np.uint16), ref_k.view(np.uint16))
    assert np.array_equal(got_v.view(np.uint16), ref_v.view(np.uint16))
    # empty calls and error behaviour
    import argus_hip as A
    assert ctx().quant_dequant_flush(qk, dev_k, hkv, d, 0, 0, 0, bits, True) == 0
    assert ctx().quant_scatter_residual(rk, dev_k, hkv, R, d, 0, 0) == 0
    assert ctx().quant_dequant_flush(qk, dev_k, hkv, d, 1, 0, 0, 3, True, check=False) == A.ERR_UNSUPPORTED
    assert ctx().quant_scatter_residual(rk, dev_k, hkv, R, d, R + 1, 0, check=False) == A.ERR_INVALID


@pytest.mark.parametrize("old,new", [(8, 4), (4, 2), (8, 2), (2, 4), (2, 8), (4, 8), (8, 8)])
def test_requant_bit_exact(old, new):
    # transition_bits between quantised widths on the device (quant_window_cache.rs:1350-1362):
    # the new stream is the CPU loop's, byte for byte.
    import torch
    rng = np.random.default_rng(500 + 10 * old + new)
    n = 4099
    src = rng.standard_normal((n, 32)).astype(np.float32)
    src[::13, 3] *= 30.0
    src[5] = -1.5                                   # constant block
    src[6] = np.round(src[6] * 2) / 2               # rounding ties
    blocks = np.concatenate([O.kivi_quantize_block(src[i], old) for i in range(n)])
    dst = torch.zeros(n * O.kivi_block_bytes(new), dtype=torch.uint8, device="cuda")
    ctx().quant_requant(dev(blocks), dst, n, old, new)
    assert np.array_equal(host(dst), O.kivi_requant(blocks, old, new))


def test_requant_argument_errors():
    import argus_hip as A
    import torch
    buf = torch.zeros(4096, dtype=torch.uint8, device="cuda")
    assert ctx().quant_requant(buf, buf[2048:], 10, 3, 4, check=False) == A.ERR_UNSUPPORTED
    assert ctx().quant_requant(buf, buf[36:], 10, 8, 4, check=False) == A.ERR_INVALID      # overlapping streams
    assert ctx().quant_requant(buf, buf[2:], 0, 8, 4, check=False) == A.OK                  # nothing to do
    assert ctx().quant_requant(buf, buf[2050:], 10, 8, 4, check=False) == A.ERR_INVALID     # misaligned


class _Raw:
    """A raw device pointer dressed as a tensor for the ctypes wrappers."""

    def __init__(self, ptr, dtype):
        self.ptr, self.dtype = ptr, dtype

    def data_ptr(self):
        return self.ptr or 0


def _read_dev(ptr, nbytes):
    import argus_hip as A
    out = np.zeros(nbytes, np.uint8)
    assert A.lib.argus_hip_read_buffer(ctx().handle, None, out.ctypes.data, ptr, nbytes) == 0
    return out


@pytest.mark.parametrize("bits", [2, 4, 8])
def test_quant_cache_capability_through_the_c_abi(bits):
    # The container behind the CACHE-category vtable (extension-api lib.rs:1932-2090) driven as the
    # layer loop drives it: a prefill update that crosses a flush, then a token per step.  Blocks and
    # residual ring against the CPU container bit for bit; fused attention over the raw buffers and the
    # F16 view against the oracle; a width transition against the oracle's requantised streams.
    import argus_hip as A
    import torch
    hq, hkv, d, R, max_seq = 8, 2, 128, 64, 400
    rng = np.random.default_rng(900 + bits)
    total = 3 * R + 21
    k = rng.standard_normal((total, hkv, d)).astype(np.float32)
    v = rng.standard_normal((total, hkv, d)).astype(np.float32)
    k[:, 1, 9] *= 15.0
    q = rng.standard_normal((hq, d)).astype(np.float32)
    kd, vd, qd = dev(k), dev(v), dev(q)
    assert ctx().quant_cache(hkv, d, max_seq, R, 3) is None            # widths 2, 4, 8 and 16 only
    assert ctx().quant_cache(hkv, d, max_seq, 48, bits) is None        # residual_size must be a multiple of 32
    c = ctx().quant_cache(hkv, d, max_seq, R, bits)
    assert c is not None and c.current_pos() == 0 and c.capacity() == max_seq and c.current_bits() == bits
    assert c.get_raw_buffers() is None                                  # empty cache: no native set
    bb = O.kivi_block_bytes(bits)

    def check_at(n, cur_bits, ref=None):
        ref = ref or O.kivi_build(k[:n], v[:n], R, cur_bits)
        assert c.current_pos() == n
        raw = c.get_raw_buffers()
        assert raw is not None and (raw.q_tokens, raw.res_tokens, raw.res_cap, raw.bits) == (ref["q_tokens"], ref["res_tokens"], R, cur_bits)
        used = ref["q_tokens"] * hkv * d // 32 * O.kivi_block_bytes(cur_bits)
        if used:
            assert np.array_equal(_read_dev(raw.qk_mem, used), ref["qk"][:used]), "key blocks (n %d)" % n
            assert np.array_equal(_read_dev(raw.qv_mem, used), ref["qv"][:used]), "value blocks (n %d)" % n
        ring = _read_dev(raw.res_k_mem, hkv * R * d * 4).view(np.float32).reshape(hkv, R, d)
        assert np.array_equal(ring[:, :ref["res_tokens"]], ref["res_k"][:, :ref["res_tokens"]])
        out = torch.empty((hq, d), device="cuda")
        sh = np.full((hq, n), -1.0, np.float32)
        ctx().attention_gen_quant(qd, _Raw(raw.qk_mem, torch.uint8), _Raw(raw.qv_mem, torch.uint8), _Raw(raw.res_k_mem, torch.float32),
                                  _Raw(raw.res_v_mem, torch.float32), out, hkv, raw.q_tokens, raw.res_tokens, raw.res_cap,
                                  1.0 / np.sqrt(d), cur_bits, scores_host=sh)
        ro, rs = O.kivi_attention(q, ref, 1.0 / np.sqrt(d), scores=True)
        check_attention_out(host(out), ro)
        check_scores(sh, rs)
        view = c.assemble_view()
        assert view.tokens == n and view.layout == 0
        gk = _read_dev(view.k_mem, n * hkv * d * 2).view(np.float16).reshape(n, hkv, d).astype(np.float32)
        gv = _read_dev(view.v_mem, n * hkv * d * 2).view(np.float16).reshape(n, hkv, d).astype(np.float32)
        ak, av = O.kivi_assemble_view(ref)
        assert np.array_equal(gk, ak.astype(np.float16).astype(np.float32)) and np.array_equal(gv, av.astype(np.float16).astype(np.float32))
        return ref

    c.update(kd[:100], vd[:100])                    # fills the ring, flushes 64, leaves 36
    check_at(100, bits)
    for t in range(100, total):
        c.update(kd[t:t + 1], vd[t:t + 1])
        if t + 1 in (128, 129, 3 * R):
            check_at(t + 1, bits)
    ref = check_at(total, bits)
    # a full ring is flushed on request, a partly filled one is left alone
    assert c.flush_if_full() == 0 and c.current_pos() == total and c.get_raw_buffers().res_tokens == ref["res_tokens"]
    # width transitions: same blocks as the CPU loop, and the cache keeps working at the new width
    for nb in [b for b in (4, 2, 8) if b != bits]:
        old = c.current_bits()
        assert c.transition_bits(nb) == 0 and c.current_bits() == nb
        ref = dict(ref, qk=O.kivi_requant(ref["qk"], old, nb), qv=O.kivi_requant(ref["qv"], old, nb), bits=nb)
        check_at(total, nb, ref)
    assert c.transition_bits(c.current_bits()) == 0                     # no-op
    assert c.transition_bits(5, check=False) == A.ERR_UNSUPPORTED
    assert c.update(dev(np.zeros((max_seq, hkv, d), np.float32)), dev(np.zeros((max_seq, hkv, d), np.float32)), check=False) == A.ERR_INVALID
    c.close()
    e = ctx().quant_cache(hkv, d, max_seq, R, 8)                        # test_kivi_transition_empty: no tokens, just the format
    assert e.transition_bits(2) == 0 and e.current_bits() == 2 and e.current_pos() == 0
    e.close()


def _flushed_ring_of_32(k, v, bits):
    """What a container with a ring of 32 tokens holds once every full group has been flushed: the
    state after transition_bits(16 -> bits).  (A dummy token triggers the lazy flush of a full ring
    and is dropped again.)"""
    n, hkv, d = k.shape
    if n % 32 == 0 and n > 0:
        z = np.zeros((1, hkv, d), np.float32)
        ref = O.kivi_build(np.concatenate([k, z]), np.concatenate([v, z]), 32, bits)
        assert ref["q_tokens"] == n and ref["res_tokens"] == 1
        ref["res_tokens"] = 0
        return ref
    return O.kivi_build(k, v, 32, bits)


@pytest.mark.parametrize("bits", [2, 4, 8])
@pytest.mark.parametrize("n", [32 * 5 + 9, 32 * 4, 7])
def test_quant_cache_unquantised_mode_and_its_transitions(bits, n):
    # bits = 16 (engine/src/kv/quant_window_cache.rs:292-300, 845-848, 2417-2429; tests 3695-3900):
    # the residual spans max_seq_len and is the view, nothing is flushed, no raw-buffer set.
    # 16 -> b quantises every full group and goes on with a ring of 32 (1137-1306); b -> 16 refills the
    # residual from the F16 view (988-1034).  Blocks bit for bit against the CPU container with a ring
    # of 32, views against the oracle's.
    import torch
    hq, hkv, d, max_seq = 8, 2, 128, 320
    rng = np.random.default_rng(1600 + bits + n)
    k = rng.standard_normal((n + 40, hkv, d)).astype(np.float32)
    v = rng.standard_normal((n + 40, hkv, d)).astype(np.float32)
    k[:, 1, 9] *= 15.0
    q = rng.standard_normal((hq, d)).astype(np.float32)
    kd, vd, qd = dev(k), dev(v), dev(q)
    c = ctx().quant_cache(hkv, d, max_seq, 64, 16)
    assert c is not None and c.current_bits() == 16 and c.capacity() == max_seq
    c.update(kd[:n], vd[:n])
    assert c.current_pos() == n and c.flush_if_full() == 0 and c.current_pos() == n
    assert c.get_raw_buffers() is None
    view = c.assemble_view()
    assert view.tokens == n and view.layout == 1
    rk = _read_dev(view.k_mem, hkv * max_seq * d * 4).view(np.float32).reshape(hkv, max_seq, d)
    rv = _read_dev(view.v_mem, hkv * max_seq * d * 4).view(np.float32).reshape(hkv, max_seq, d)
    assert np.array_equal(rk[:, :n], k[:n].transpose(1, 0, 2)) and np.array_equal(rv[:, :n], v[:n].transpose(1, 0, 2))
    assert c.transition_bits(16) == 0                                    # no-op

    def check_quantised(ref, n_now, cur_bits):
        raw = c.get_raw_buffers()
        assert c.current_pos() == n_now and c.current_bits() == cur_bits
        if n_now == 0:
            assert raw is None
            return
        assert (raw.q_tokens, raw.res_tokens, raw.res_cap, raw.bits) == (ref["q_tokens"], ref["res_tokens"], 32, cur_bits)
        used = ref["q_tokens"] * hkv * d // 32 * O.kivi_block_bytes(cur_bits)
        if used:
            assert np.array_equal(_read_dev(raw.qk_mem, used), ref["qk"][:used]), "key blocks"
            assert np.array_equal(_read_dev(raw.qv_mem, used), ref["qv"][:used]), "value blocks"
        ring = _read_dev(raw.res_k_mem, hkv * 32 * d * 4).view(np.float32).reshape(hkv, 32, d)
        assert np.array_equal(ring[:, :ref["res_tokens"]], ref["res_k"][:, :ref["res_tokens"]])
        out = torch.empty((hq, d), device="cuda")
        ctx().attention_gen_quant(qd, _Raw(raw.qk_mem, torch.uint8), _Raw(raw.qv_mem, torch.uint8), _Raw(raw.res_k_mem, torch.float32),
                                  _Raw(raw.res_v_mem, torch.float32), out, hkv, raw.q_tokens, raw.res_tokens, raw.res_cap,
                                  1.0 / np.sqrt(d), cur_bits)
        check_attention_out(host(out), O.kivi_attention(q, ref, 1.0 / np.sqrt(d)))
        vw = c.assemble_view()
        assert vw.tokens == n_now and vw.layout == 0
        gk = _read_dev(vw.k_mem, n_now * hkv * d * 2).view(np.float16).reshape(n_now, hkv, d)
        ak, av = O.kivi_assemble_view(ref)
        assert np.array_equal(gk, ak.astype(np.float16))

    # 16 -> b
    assert c.transition_bits(bits) == 0
    ref = _flushed_ring_of_32(k[:n], v[:n], bits)
    check_quantised(ref, n, bits)
    # the cache keeps working with its ring of 32: forty more tokens, one at a time
    for t in range(n, n + 40):
        c.update(kd[t:t + 1], vd[t:t + 1])
    ref = O.kivi_build(k[:n + 40], v[:n + 40], 32, bits)
    if n % 32 == 0:  # the transition flushed a ring the lazy rule would have kept full for one more token
        assert ref["q_tokens"] == c.get_raw_buffers().q_tokens
    check_quantised(ref, n + 40, bits)
    # b -> 16: every token back in the residual, through the F16 view
    ak, av = O.kivi_assemble_view(ref)
    assert c.transition_bits(16) == 0 and c.current_bits() == 16 and c.current_pos() == n + 40
    assert c.get_raw_buffers() is None
    view = c.assemble_view()
    assert view.tokens == n + 40 and view.layout == 1
    rk = _read_dev(view.k_mem, hkv * max_seq * d * 4).view(np.float32).reshape(hkv, max_seq, d)[:, :n + 40]
    rv = _read_dev(view.v_mem, hkv * max_seq * d * 4).view(np.float32).reshape(hkv, max_seq, d)[:, :n + 40]
    k16 = ak.astype(np.float16).astype(np.float32).transpose(1, 0, 2)
    v16 = av.astype(np.float16).astype(np.float32).transpose(1, 0, 2)
    assert np.array_equal(rk, k16) and np.array_equal(rv, v16)
    # and down again at another width, from the restored values
    nb = 4 if bits != 4 else 8
    assert c.transition_bits(nb) == 0
    ref2 = _flushed_ring_of_32(np.ascontiguousarray(k16.transpose(1, 0, 2)), np.ascontiguousarray(v16.transpose(1, 0, 2)), nb)
    check_quantised(ref2, n + 40, nb)
    c.close()
    e = ctx().quant_cache(hkv, d, max_seq, 64, 16)                       # empty cache: only the format changes
    assert e.transition_bits(bits) == 0 and e.current_bits() == bits and e.current_pos() == 0 and e.get_raw_buffers() is None
    e.update(kd[:3], vd[:3])
    assert e.get_raw_buffers().res_cap == 32 and e.transition_bits(16) == 0 and e.assemble_view().tokens == 3
    e.close()


def test_quant_cache_make_refuses_a_foreign_context_and_another_stream():
    # the ctx slot of the make arguments is untyped (the reference's cl_context): only this library's
    # contexts are accepted; and a handle works on the stream it was made with
    import argus_hip as A
    import torch
    junk = (C.c_uint64 * 64)(*([0x1234567890] * 64))
    a = A.QuantCacheMakeArgs(ctx=C.addressof(junk), device=None, stream=None, build_opts=None, kv_heads=2, head_dim=64,
                             max_seq_len=128, residual_size=32, bits=4)
    assert not A.lib.argus_hip_quant_cache_make(C.byref(a))
    c = ctx().quant_cache(2, 64, 128, 32, 4)
    x = torch.zeros((1, 2, 64), device="cuda")
    other = torch.cuda.Stream()
    u = A.QuantCacheUpdateArgs(stream=other.cuda_stream, k_in_mem=x.data_ptr(), v_in_mem=x.data_ptr(), seq_len=1)
    assert A.lib.argus_hip_quant_cache_update(c.handle, C.byref(u)) == A.ERR_INVALID
    c.update(x, x)
    assert c.current_pos() == 1
    c.close()


def test_plugin_protocol_end_to_end():
    # What engine/src/capability/dynamic_backend_registry.rs does with a capability plugin: dlopen,
    # register_backend_caps_v2, pick the entries by name, call through the vtables only.  The CACHE
    # handle builds a cache from tokens on the device, the ATTENTION handle attends over its raw buffers.
    import argus_hip as A
    import torch
    env = A.lib.register_backend_caps_v2()
    by_name = {env.vtables[i].name: env.vtables[i] for i in range(env.count)}
    attn = C.cast(by_name[b"kivi_hip"].vtable, C.POINTER(A.QuantAttnVTable)).contents
    cache = C.cast(by_name[b"kivi_cache_hip"].vtable, C.POINTER(A.QuantCacheVTable)).contents
    vp = C.c_void_p
    a_make = C.CFUNCTYPE(vp, C.POINTER(A.QuantAttnMakeArgs))(attn.make)
    a_has = C.CFUNCTYPE(C.c_bool, vp, C.c_uint8)(attn.has_quant_attn_kernel)
    a_nosub = C.CFUNCTYPE(C.c_bool, vp)(attn.is_nosub_device)
    a_attn = C.CFUNCTYPE(C.c_int32, vp, C.POINTER(A.QuantAttnArgs))(attn.attention_gen_quant)
    a_drop = C.CFUNCTYPE(None, vp)(attn.drop)
    c_make = C.CFUNCTYPE(vp, C.POINTER(A.QuantCacheMakeArgs))(cache.make)
    c_update = C.CFUNCTYPE(C.c_int32, vp, C.POINTER(A.QuantCacheUpdateArgs))(cache.update)
    c_pos = C.CFUNCTYPE(C.c_size_t, vp)(cache.current_pos)
    c_raw = C.CFUNCTYPE(C.c_bool, vp, C.POINTER(A.QuantCacheRawBuffersOut))(cache.get_raw_buffers)
    c_drop = C.CFUNCTYPE(None, vp)(cache.drop)

    hq, hkv, d, R, n, bits = 8, 2, 128, 32, 75, 4
    rng = np.random.default_rng(4242)
    k = rng.standard_normal((n, hkv, d)).astype(np.float32)
    v = rng.standard_normal((n, hkv, d)).astype(np.float32)
    q = rng.standard_normal((hq, d)).astype(np.float32)
    kd, vd, qd = dev(k), dev(v), dev(q)
    stream = torch.cuda.current_stream().cuda_stream
    ah = a_make(C.byref(A.QuantAttnMakeArgs()))          # the OpenCL handles of the reference are not used
    assert ah and a_has(ah, 2) and a_has(ah, 4) and a_has(ah, 8) and not a_has(ah, 3) and a_nosub(ah)
    ch = c_make(C.byref(A.QuantCacheMakeArgs(ctx=None, stream=stream, kv_heads=hkv, head_dim=d, max_seq_len=128, residual_size=R, bits=bits)))
    assert ch
    assert c_update(ch, C.byref(A.QuantCacheUpdateArgs(stream=stream, k_in_mem=kd.data_ptr(), v_in_mem=vd.data_ptr(), seq_len=n))) == 0
    assert c_pos(ch) == n
    raw = A.QuantCacheRawBuffersOut()
    assert c_raw(ch, C.byref(raw)) and (raw.q_tokens, raw.res_tokens, raw.bits) == (64, 11, bits)
    out = torch.empty((hq, d), device="cuda")
    sh = np.zeros((hq, n), np.float32)
    args = A.QuantAttnArgs(stream=stream, q_mem=qd.data_ptr(), qk_mem=raw.qk_mem, qv_mem=raw.qv_mem, res_k_mem=raw.res_k_mem,
                           res_v_mem=raw.res_v_mem, out_mem=out.data_ptr(), scores_out=sh.ctypes.data, scores_len=sh.size,
                           num_heads_q=hq, num_heads_kv=hkv, head_dim=d, q_tokens=raw.q_tokens, res_tokens=raw.res_tokens,
                           res_cap=raw.res_cap, scale=1.0 / np.sqrt(d), bits=bits)
    assert a_attn(ah, C.byref(args)) == 0
    ref = O.kivi_build(k, v, R, bits)
    ro, rs = O.kivi_attention(q, ref, 1.0 / np.sqrt(d), scores=True)
    check_attention_out(host(out), ro)
    check_scores(sh, rs)
    args.bits = 3
    assert a_attn(ah, C.byref(args)) < 0
    c_drop(ch)
    a_drop(ah)
