"""Committed fixtures (tests/golden/*.npz, written by tests/golden/make_golden.py): the oracle must still
reproduce them bit for bit (CPU), and the HIP library must match them (GPU)."""
import os

import numpy as np
import pytest

import oracle as O

G = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def load(name):
    return dict(np.load(os.path.join(G, name + ".npz")))


def bits_equal(a, b):
    a, b = np.ascontiguousarray(a), np.ascontiguousarray(b)
    return a.shape == b.shape and a.dtype == b.dtype and np.array_equal(a.view(np.uint8), b.view(np.uint8))


# ---- CPU: the oracle against the fixtures --------------------------------------------------------
def test_oracle_decode_reproduces_fixture():
    f = load("decode_f16")
    hq, hkv, d, L, cap = f["dims"]
    out, sc = O.attention_gen(f["q"], f["k"], f["v"], hkv, L, cap, scores=True)
    assert bits_equal(out, f["out"]) and bits_equal(sc, f["scores"])
    out, sc = O.attention_gen(f["q"], f["k"], f["v"], hkv, L, cap, scores=True, softcap=5.0)
    assert bits_equal(out, f["out_softcap5"]) and bits_equal(sc, f["scores_softcap5"])
    # the AVX2 restatement agrees with the scalar one within the reference's own bound
    out2 = O.attention_gen(f["q"], f["k"], f["v"], hkv, L, cap, impl="avx2")
    assert np.abs(out2 - f["out"]).max() < 1e-3


def test_oracle_prefill_reproduces_fixture():
    f = load("prefill_f32")
    hq, hkv, d, S, C, cap = f["dims"]
    assert bits_equal(O.prefill_attention(f["q"], f["k"], f["v"], hkv, C, cap, n_threads=1), f["out"])


@pytest.mark.parametrize("bits", [2, 4, 8])
def test_oracle_kivi_reproduces_fixture(bits):
    f = load("kivi")
    hq, hkv, d, R, n = f["dims"]
    c = O.kivi_build(f["k_tokens"], f["v_tokens"], R, bits)
    assert bits_equal(c["qk"], f["qk%d" % bits]) and bits_equal(c["qv"], f["qv%d" % bits])
    assert bits_equal(c["res_k"], f["res_k"]) and [c["q_tokens"], c["res_tokens"]] == list(f["q_res_tokens"])
    out, sc = O.kivi_attention(f["q"], c, 1.0 / np.sqrt(d), scores=True)
    assert bits_equal(out, f["out%d" % bits]) and bits_equal(sc, f["scores%d" % bits])


def test_oracle_reduce_pfa_descriptor_reproduce_fixtures():
    f = load("score_reduce")
    n_layers, hq, hkv, L, stride = f["dims"]
    imp, himp = f["importance_in"].copy(), f["head_importance_in"].copy()
    O.score_fused_reduce(f["scores"], imp, himp, 0.9, n_layers, hq, hkv, L, stride, stride)
    assert bits_equal(imp, f["importance_out"]) and bits_equal(himp, f["head_importance_out"])
    f = load("pfa")
    nq, nkv, d, S, prefix, qs, qw = f["dims"]
    s = np.zeros((nq, prefix), np.float32)
    ph = np.zeros((qw, nq, prefix), np.float32)
    O.prefill_attention_scores(f["q"], f["k"], nq, nkv, d, S, prefix, nkv * d, d, qs, qw, None, sum_out=s, per_row=ph,
                               per_head=True)
    assert bits_equal(s, f["sum_out"]) and bits_equal(ph, f["per_head"])
    f = load("descriptor")
    assert bits_equal(O.encode_via_descriptor(O.DESC_Q4_0, f["x"]), f["q4_0"])
    assert bits_equal(O.encode_via_descriptor(O.DESC_Q2_0, f["x"]), f["q2_0"])
    assert bits_equal(O.decode_via_descriptor(O.DESC_Q4_0, f["q4_0"], f["x"].size), f["q4_0_decoded"])


# ---- GPU: the library against the fixtures -------------------------------------------------------
@pytest.mark.gpu
def test_gpu_decode_matches_fixture():
    import torch
    from gpu_util import check_attention_out, check_scores, ctx, dev, host
    f = load("decode_f16")
    hq, hkv, d, L, cap = (int(x) for x in f["dims"])
    for softcap, ko, ks in ((0.0, "out", "scores"), (5.0, "out_softcap5", "scores_softcap5")):
        out = torch.zeros((hq, d), device="cuda")
        sc = torch.zeros((hq, L), device="cuda")
        ctx().attention_gen(dev(f["q"]), dev(f["k"]), dev(f["v"]), out, hkv, L, cap, scores=sc, score_stride=L, softcap=softcap)
        check_attention_out(host(out), f[ko])
        check_scores(host(sc), f[ks])


@pytest.mark.gpu
def test_gpu_prefill_matches_fixture():
    import torch
    from gpu_util import check_attention_out, ctx, dev, host
    f = load("prefill_f32")
    hq, hkv, d, S, C, cap = (int(x) for x in f["dims"])
    out = torch.zeros((1, S, hq, d), device="cuda")
    assert ctx().flash_attention_prefill(dev(f["q"]), dev(f["k"]), dev(f["v"]), out, hq, hkv, S, C, d, cap) == 1
    check_attention_out(host(out), f["out"])


@pytest.mark.gpu
@pytest.mark.parametrize("bits", [2, 4, 8])
def test_gpu_kivi_matches_fixture(bits):
    import torch
    from gpu_util import check_attention_out, check_scores, ctx, dev, host
    f = load("kivi")
    hq, hkv, d, R, n = (int(x) for x in f["dims"])
    qt, rt = (int(x) for x in f["q_res_tokens"])
    out = torch.zeros((hq, d), device="cuda")
    sc = torch.zeros((hq, n), device="cuda")
    ctx().attention_gen_quant(dev(f["q"]), dev(f["qk%d" % bits]), dev(f["qv%d" % bits]), dev(f["res_k"]), dev(f["res_v"]), out,
                              hkv, qt, rt, R, 1.0 / np.sqrt(d), bits, scores_dev=sc, score_stride=n)
    check_attention_out(host(out), f["out%d" % bits])
    check_scores(host(sc), f["scores%d" % bits])
    # on-device quantise-at-flush reproduces the fixture's blocks bit for bit (first flush of R tokens)
    rk = np.ascontiguousarray(f["k_tokens"][:R].transpose(1, 0, 2))
    rv = np.ascontiguousarray(f["v_tokens"][:R].transpose(1, 0, 2))
    bb = O.kivi_block_bytes(bits)
    nk = hkv * (R // 32) * d
    qk = torch.zeros(nk * bb, device="cuda", dtype=torch.uint8)
    qv = torch.zeros(nk * bb, device="cuda", dtype=torch.uint8)
    ctx().quant_flush(dev(rk), dev(rv), qk, qv, hkv, R, d, R, 0, 0, bits)
    assert np.array_equal(host(qk), f["qk%d" % bits][:nk * bb]) and np.array_equal(host(qv), f["qv%d" % bits][:nk * bb])


@pytest.mark.gpu
def test_gpu_reduce_pfa_descriptor_match_fixtures():
    import torch
    from gpu_util import check_scores, ctx, dev, host
    f = load("score_reduce")
    n_layers, hq, hkv, L, stride = (int(x) for x in f["dims"])
    imp, himp = dev(f["importance_in"]), dev(f["head_importance_in"])
    ctx().score_reduce(dev(f["scores"]), imp, himp, 0.9, n_layers, hq, hkv, L, stride, stride)
    assert np.allclose(host(imp), f["importance_out"], rtol=1e-6, atol=1e-7)
    assert np.allclose(host(himp), f["head_importance_out"], rtol=1e-6, atol=1e-7)
    f = load("pfa")
    nq, nkv, d, S, prefix, qs, qw = (int(x) for x in f["dims"])
    s = torch.zeros((nq, prefix), device="cuda")
    ph = torch.zeros((qw, nq, prefix), device="cuda")
    ctx().prefill_attention_scores(dev(f["q"]), dev(f["k"]), nq, nkv, d, S, prefix, nkv * d, d, qs, qw, None, sum_out=s,
                                   per_row=ph, per_head=True)
    check_scores(host(s), f["sum_out"])
    check_scores(host(ph), f["per_head"])
    f = load("descriptor")
    n = f["x"].size
    q4 = torch.zeros(f["q4_0"].size, device="cuda", dtype=torch.uint8)
    q2 = torch.zeros(f["q2_0"].size, device="cuda", dtype=torch.uint8)
    ctx().kv_encode_descriptor(O.DESC_Q4_0, dev(f["x"]), q4, n)
    ctx().kv_encode_descriptor(O.DESC_Q2_0, dev(f["x"]), q2, n)
    assert np.array_equal(host(q4), f["q4_0"]) and np.array_equal(host(q2), f["q2_0"])
    back = torch.zeros(n, device="cuda")
    ctx().kv_decode_descriptor(O.DESC_Q4_0, q4, back, n)
    assert np.array_equal(host(back).view(np.uint32), f["q4_0_decoded"].view(np.uint32))


def test_oracle_block_attention_reproduces_fixture():
    f = load("blocks")
    hq, hkv, d, L, cap = [int(x) for x in f["dims"]]
    for fmt, desc in (("q4_0", O.DESC_Q4_0), ("q8_0", O.DESC_Q8_0), ("q2_0", O.DESC_Q2_0)):
        out, sc = O.attention_gen_blocks(f["q"], f["k_" + fmt], f["v_" + fmt], desc, hkv, L, cap, scores=True)
        assert bits_equal(out, f["out_" + fmt]) and bits_equal(sc, f["scores_" + fmt])


@pytest.mark.gpu
def test_gpu_block_attention_matches_fixture():
    import argus_hip as A
    from gpu_util import ctx, dev, host, check_attention_out, check_scores
    f = load("blocks")
    hq, hkv, d, L, cap = [int(x) for x in f["dims"]]
    for fmt, code in (("q4_0", A.Q4_0), ("q8_0", A.Q8_0), ("q2_0", A.Q2_0)):
        out = dev(np.zeros((hq, d), np.float32))
        sc = dev(np.zeros((hq, L), np.float32))
        ctx().attention_gen(dev(f["q"]), dev(f["k_" + fmt]), dev(f["v_" + fmt]), out, hkv, L, cap, scores=sc,
                            score_stride=L, kv_dtype=code)
        check_attention_out(host(out), f["out_" + fmt], fmt)
        check_scores(host(sc), f["scores_" + fmt], fmt)
