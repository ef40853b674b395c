"""GPU parity: score reduce, KV scatter and the post-eviction + H2O flow (benchmark configuration 5)."""
import numpy as np
import pytest

import oracle as O
import textbook as T
from gpu_util import check_attention_out, check_scores, ctx, dev, host, normal

pytestmark = pytest.mark.gpu


def f16(x):
    return O.f32_to_f16_bits(x).view(np.float16)


def test_score_reduce_known_answers():
    # engine/src/bin/test_cuda_gpu_score_device.rs cases 1 and 2.
    import torch
    nl, hq, hkv, max_seq, L = 2, 2, 1, 8, 3
    sc = np.zeros((nl, hq, max_seq), np.float32)
    sc[0, 0, :3], sc[0, 1, :3] = [0.1, 0.2, 0.7], [0.3, 0.3, 0.4]
    sc[1, 0, :3], sc[1, 1, :3] = [0.5, 0.4, 0.1], [0.2, 0.2, 0.6]
    s = dev(sc)
    imp = torch.zeros(max_seq, device="cuda")
    himp = torch.zeros(hkv * max_seq, device="cuda")
    ctx().score_reduce(s, imp, himp, 1.0, nl, hq, hkv, L, max_seq, max_seq)
    assert np.abs(host(imp)[:3] - [0.7, 0.6, 1.1]).max() < 1e-5
    assert np.abs(host(himp)[:3] - [0.35, 0.30, 0.55]).max() < 1e-5
    assert not host(imp)[3:].any()
    imp.zero_()
    himp.zero_()
    for _ in range(2):
        ctx().score_reduce(s, imp, himp, 0.5, nl, hq, hkv, L, max_seq, max_seq)
    assert np.abs(host(imp)[:3] - 1.5 * np.array([0.7, 0.6, 1.1])).max() < 1e-5
    lf = torch.zeros(nl * max_seq, device="cuda")
    ctx().score_reduce_per_layer(s, lf, 1.0, nl, hq, hkv, L, max_seq, max_seq)
    assert np.abs(host(lf)[:3] - [0.4, 0.5, 1.1]).max() < 1e-6
    assert np.abs(host(lf)[8:11] - [0.7, 0.6, 0.7]).max() < 1e-6


@pytest.mark.parametrize("nl,hq,hkv,L,stride", [(1, 8, 4, 2048, 4096), (28, 14, 2, 1000, 1024),
                                                (32, 32, 8, 4097, 8192), (3, 16, 16, 70, 70)])
def test_score_reduce_vs_oracle(nl, hq, hkv, L, stride):
    import torch
    rng = np.random.default_rng(nl * 1000 + L)
    sc = rng.random((nl, hq, stride), dtype=np.float32)
    imp0 = rng.random(stride, dtype=np.float32)
    himp0 = rng.random(hkv * stride, dtype=np.float32)
    lf0 = rng.random(nl * stride, dtype=np.float32)
    imp, himp, lf = imp0.copy(), himp0.copy(), lf0.copy()
    O.score_fused_reduce(sc, imp, himp, 0.9, nl, hq, hkv, L, stride, stride)
    O.score_reduce_per_layer(sc, lf, 0.9, nl, hq, L, stride, stride)
    s, di, dh, dl = dev(sc), dev(imp0), dev(himp0), dev(lf0)
    ctx().score_reduce(s, di, dh, 0.9, nl, hq, hkv, L, stride, stride)
    ctx().score_reduce_per_layer(s, dl, 0.9, nl, hq, hkv, L, stride, stride)
    assert np.allclose(host(di), imp, rtol=1e-5, atol=0)
    assert np.allclose(host(dh), himp, rtol=1e-5, atol=0)
    assert np.allclose(host(dl), lf, rtol=1e-5, atol=0)
    # untouched beyond cache_seq_len
    assert np.array_equal(host(di)[L:], imp0[L:])
    import argus_hip as A
    assert ctx().score_reduce(s, di, dh, 0.9, nl, hq, 17, L, stride, stride, check=False) < 0


@pytest.mark.parametrize("seq_len,write_pos", [(1, 0), (1, 37), (64, 10), (2048, 0)])
@pytest.mark.parametrize("to_f16", [True, False])
def test_kv_scatter(seq_len, write_pos, to_f16):
    import torch
    hkv, d, cap = 8, 128, 2100
    ks = normal((seq_len, hkv, d), 1) * 3
    vs = normal((seq_len, hkv, d), 2) * 3
    dt = np.float16 if to_f16 else np.float32
    kd = np.full((hkv, cap, d), 7, dt)
    vd = np.full((hkv, cap, d), 7, dt)
    dk, dv = dev(kd), dev(vd)
    ctx().kv_scatter(dev(ks), dev(vs), dk, dv, hkv, d, cap, write_pos,
                     seq_len=None if (seq_len == 1 and to_f16) else seq_len)
    O.kv_scatter(ks, vs, kd, vd, write_pos)
    assert np.array_equal(host(dk).view(np.uint16 if to_f16 else np.uint32),
                          kd.view(np.uint16 if to_f16 else np.uint32))
    assert np.array_equal(host(dv).view(np.uint16 if to_f16 else np.uint32),
                          vd.view(np.uint16 if to_f16 else np.uint32))
    import argus_hip as A
    assert ctx().kv_scatter(dev(ks), dev(vs), dk, dv, hkv, d, cap, cap, seq_len=seq_len, check=False) == A.ERR_INVALID


@pytest.mark.parametrize("batch", [1, 8])
@pytest.mark.parametrize("softcap", [50.0, 0.0])
def test_config5_post_eviction_h2o_flow(batch, softcap):
    # benchmark configuration 5 (Gemma-2-2B shape): 8192-token history compacted StreamingLLM-style
    # (sink 4 + recent 2044 -> kept positions {0..3} U {6148..8191}, 2048 valid slots) into a
    # capacity-4096 HeadMajor cache; decode with soft-cap 50; per-position probabilities are
    # emitted and reduced to H2O importance.  soft-cap 0 is the reference-CPU-semantics variant.
    import torch
    hq, hkv, d, hist, cap = 8, 4, 256, 8192, 4096
    keep = O.streaming_keep(4, 2044, hist, 0)
    L = len(keep)
    assert L == 2048
    q = normal((batch, hq, d), 42)
    kc = np.zeros((batch, hkv, cap, d), np.float16)
    vc = np.zeros((batch, hkv, cap, d), np.float16)
    for b in range(batch):
        kh = f16(normal((hkv, hist, d), 137 + b))
        vh = f16(normal((hkv, hist, d), 53 + b))
        kc[b] = O.compact_keep(kh, keep, cap)
        vc[b] = O.compact_keep(vh, keep, cap)
    out = torch.empty((batch, hq, d), device="cuda")
    sc = torch.zeros((batch, hq, cap), device="cuda")
    ctx().attention_gen(dev(q), dev(kc), dev(vc), out, hkv, L, cap, scores=sc, score_stride=cap,
                        batch=batch, kv_batch_stride=hkv * cap * d, softcap=softcap)
    got, gsc = host(out), host(sc)
    for b in range(batch):
        ref, p = O.attention_gen(q[b], kc[b], vc[b], hkv, L, cap, scores=True, scores_stride=cap,
                                 softcap=softcap)
        check_attention_out(got[b], ref, "seq %d" % b)
        check_scores(gsc[b, :, :L], p[:, :L], "seq %d" % b)
        # fused reduce (single layer) on the device score buffer of this sequence
        imp = torch.zeros(cap, device="cuda")
        himp = torch.zeros(hkv * cap, device="cuda")
        ctx().score_reduce(sc[b], imp, himp, 1.0, 1, hq, hkv, L, cap, cap)
        oi, oh = np.zeros(cap, np.float32), np.zeros(hkv * cap, np.float32)
        O.score_fused_reduce(p, oi, oh, 1.0, 1, hq, hkv, L, cap, cap)
        check_scores(host(imp), oi, "importance")
        check_scores(host(himp), oh, "head importance")
        flat, head = T.score_reduce(T.decode_attention(q[b], kc[b], vc[b], hkv, L, softcap=softcap)[1][None], hkv)
        check_scores(host(imp)[:L], flat, "importance vs f64")


@pytest.mark.parametrize("hq,hkv,d,L,cap,softcap", [(8, 4, 256, 3000, 4096, 50.0), (32, 8, 128, 2500, 4096, 0.0)])
def test_h2o_loop_scores_to_keep_list_to_post_eviction_attention(hq, hkv, d, L, cap, softcap):
    # The loop benchmark configuration 5 feeds, closed on the device: three decode steps emit scores, the fused
    # reduce accumulates importance (decay 0) and per-KV-head importance, H2O's keep-spec
    # (crates/techniques/h2o/src/lib.rs:138-160: flat, then per head) turns them into keep-lists on
    # the host, and the next decode attends the survivors (a) through kv_index over the untouched
    # cache, (b) over a cache compacted in place on the device by the reference's runs of overlapping
    # buffer_shift moves (engine/src/kv/kv_cache.rs:1266-1350) -- both must equal the oracle's
    # gather-then-attend, and the keep-lists made from device scores must be the oracle's.
    import torch
    steps, hh, recent, prefix = 3, 256, 512, 4
    k = f16(normal((hkv, cap, d), 137))
    v = f16(normal((hkv, cap, d), 53))
    kd, vd = dev(k), dev(v)
    imp = torch.zeros(cap, device="cuda")
    himp = torch.zeros(hkv * cap, device="cuda")
    oi, oh = np.zeros(cap, np.float32), np.zeros(hkv * cap, np.float32)
    for s in range(steps):
        q = normal((hq, d), 42 + s)
        out = torch.empty((hq, d), device="cuda")
        sc = torch.zeros((hq, cap), device="cuda")
        ctx().attention_gen(dev(q), kd, vd, out, hkv, L, cap, scores=sc, score_stride=cap, softcap=softcap)
        ctx().score_reduce(sc, imp, himp, 1.0, 1, hq, hkv, L, cap, cap)
        _, p = O.attention_gen(q, k, v, hkv, L, cap, scores=True, scores_stride=cap, softcap=softcap)
        O.score_fused_reduce(p, oi, oh, 1.0, 1, hq, hkv, L, cap, cap)
    check_scores(host(imp)[:L], oi[:L], "cumulative importance")
    check_scores(host(himp).reshape(hkv, cap)[:, :L], oh.reshape(hkv, cap)[:, :L], "cumulative head importance")

    q = normal((hq, d), 99)
    # (1) flat keep-list from the layer-wide importance
    kind, keep = O.h2o_keep_spec(L, hh, recent, prefix, importance=host(imp))
    kind_o, keep_o = O.h2o_keep_spec(L, hh, recent, prefix, importance=oi)
    assert kind == kind_o == "layer" and len(keep) == prefix + hh + recent
    assert np.array_equal(keep, keep_o), "keep-list from device scores differs from the oracle's"
    n = len(keep)
    ref = O.attention_gen(q, O.compact_keep(k, keep, cap), O.compact_keep(v, keep, cap), hkv, n, cap, softcap=softcap)
    out = torch.empty((hq, d), device="cuda")
    ctx().attention_gen(dev(q), kd, vd, out, hkv, n, cap, kv_index=dev(keep.astype(np.int32)), softcap=softcap)
    check_attention_out(host(out), ref, "through kv_index")
    kc, vc = kd.clone(), vd.clone()
    for src, dst, count in O.keep_batches(keep):
        for h in range(hkv):
            base = h * cap * d
            ctx().buffer_shift(kc, base + src * d, base + dst * d, count * d)
            ctx().buffer_shift(vc, base + src * d, base + dst * d, count * d)
    assert np.array_equal(host(kc)[:, :n], k[:, keep]) and np.array_equal(host(vc)[:, :n], v[:, keep])
    ctx().attention_gen(dev(q), kc, vc, out, hkv, n, cap, softcap=softcap)
    check_attention_out(host(out), ref, "over the compacted cache")

    # (2) per-head keep-lists from the per-KV-head importance: every head compacts its own survivors
    kind, heads = O.h2o_keep_spec(L, hh, recent, prefix, head_scores=host(himp).reshape(hkv, cap))
    kind_o, heads_o = O.h2o_keep_spec(L, hh, recent, prefix, head_scores=oh.reshape(hkv, cap))
    assert kind == kind_o == "per_head"
    assert all(np.array_equal(a, b) for a, b in zip(heads, heads_o)), "per-head keep-lists differ from the oracle's"
    assert any(not np.array_equal(heads[0], h) for h in heads[1:]), "heads should rank their own heavy hitters"
    kc, vc = kd.clone(), vd.clone()
    kg, vg = np.zeros_like(k), np.zeros_like(v)
    for h in range(hkv):
        kg[h, :n], vg[h, :n] = k[h, heads[h]], v[h, heads[h]]
        base = h * cap * d
        for src, dst, count in O.keep_batches(heads[h]):
            ctx().buffer_shift(kc, base + src * d, base + dst * d, count * d)
            ctx().buffer_shift(vc, base + src * d, base + dst * d, count * d)
    assert np.array_equal(host(kc)[:, :n], kg[:, :n]) and np.array_equal(host(vc)[:, :n], vg[:, :n])
    sc = torch.zeros((hq, cap), device="cuda")
    ctx().attention_gen(dev(q), kc, vc, out, hkv, n, cap, scores=sc, score_stride=cap, softcap=softcap)
    ref, p = O.attention_gen(q, kg, vg, hkv, n, cap, scores=True, scores_stride=cap, softcap=softcap)
    check_attention_out(host(out), ref, "per-head compaction")
    check_scores(host(sc)[:, :n], p[:, :n], "scores after per-head compaction")


def _decode_both_forms(q, kc, vc, hkv, L, cap, batch, softcap=0.0, context=None):
    """One call with probabilities out, one with logits + (max, sum): (out, p, out2, logits, stats)."""
    import torch
    c = context or ctx()
    hq, d = q.shape[-2], q.shape[-1]
    qd, kd, vd = dev(q), dev(kc), dev(vc)
    out = torch.empty((batch, hq, d), device="cuda")
    sc = torch.zeros((batch, hq, cap), device="cuda")
    c.attention_gen(qd, kd, vd, out, hkv, L, cap, scores=sc, score_stride=cap, batch=batch,
                    kv_batch_stride=hkv * cap * d, softcap=softcap)
    out2 = torch.empty_like(out)
    lg = torch.zeros_like(sc)
    st = torch.zeros((batch, hq, 2), device="cuda")
    c.attention_gen(qd, kd, vd, out2, hkv, L, cap, scores=lg, score_stride=cap, batch=batch,
                    kv_batch_stride=hkv * cap * d, softcap=softcap, score_stats=st)
    return out, sc, out2, lg, st


@pytest.mark.parametrize("batch", [1, 8])
def test_config5_importance_through_the_logits_and_statistics_form(batch):
    # The opt-in score form: the attention call leaves the logits and writes (max, sum) per row, the
    # reduce normalises while it reads.  Same arithmetic as the rewrite it replaces, so the importance
    # vectors must equal the probability form's bit for bit, and the oracle's to 1e-4 relative.
    import torch
    hq, hkv, d, hist, cap, softcap = 8, 4, 256, 8192, 4096, 50.0
    keep = O.streaming_keep(4, 2044, hist, 0)
    L = len(keep)
    q = normal((batch, hq, d), 42)
    kc = np.zeros((batch, hkv, cap, d), np.float16)
    vc = np.zeros((batch, hkv, cap, d), np.float16)
    for b in range(batch):
        kc[b] = O.compact_keep(f16(normal((hkv, hist, d), 137 + b)), keep, cap)
        vc[b] = O.compact_keep(f16(normal((hkv, hist, d), 53 + b)), keep, cap)
    out, sc, out2, lg, st = _decode_both_forms(q, kc, vc, hkv, L, cap, batch, softcap)
    assert torch.equal(out, out2)
    m, l = st[..., 0:1], st[..., 1:2]
    assert torch.allclose(torch.exp(lg[..., :L] - m) / l, sc[..., :L], rtol=1e-5, atol=0)
    for b in range(batch):
        imp, himp = torch.zeros(cap, device="cuda"), torch.zeros(hkv * cap, device="cuda")
        ctx().score_reduce(sc[b], imp, himp, 1.0, 1, hq, hkv, L, cap, cap)
        imp2, himp2 = torch.zeros(cap, device="cuda"), torch.zeros(hkv * cap, device="cuda")
        ctx().score_reduce(lg[b], imp2, himp2, 1.0, 1, hq, hkv, L, cap, cap, stats=st[b])
        assert torch.equal(imp, imp2) and torch.equal(himp, himp2)
        lf, lf2 = torch.zeros(cap, device="cuda"), torch.zeros(cap, device="cuda")
        ctx().score_reduce_per_layer(sc[b], lf, 0.5, 1, hq, hkv, L, cap, cap)
        ctx().score_reduce_per_layer(lg[b], lf2, 0.5, 1, hq, hkv, L, cap, cap, stats=st[b])
        assert torch.equal(lf, lf2)
        _, p = O.attention_gen(q[b], kc[b], vc[b], hkv, L, cap, scores=True, scores_stride=cap, softcap=softcap)
        oi, oh = np.zeros(cap, np.float32), np.zeros(hkv * cap, np.float32)
        O.score_fused_reduce(p, oi, oh, 1.0, 1, hq, hkv, L, cap, cap)
        check_scores(host(imp2), oi, "importance, seq %d" % b)
        check_scores(host(himp2), oh, "head importance, seq %d" % b)


def test_config3_batch16_importance_through_the_logits_and_statistics_form():
    # 16 sequences of the Llama-3-8B head shape at 32K tokens; the 16 score buffers double as the
    # "layers" of one reduce.  Bit equality with the probability form on everything, the oracle on a
    # sampled sequence.
    import torch
    b, hq, hkv, d, L = 16, 32, 8, 128, 32768
    g = torch.Generator(device="cuda").manual_seed(137)
    k = torch.randn((b, hkv, L, d), generator=g, device="cuda", dtype=torch.float32).half()
    v = torch.randn((b, hkv, L, d), generator=g, device="cuda", dtype=torch.float32).half()
    q = dev(normal((b, hq, d), 42))
    out, out2 = torch.empty((b, hq, d), device="cuda"), torch.empty((b, hq, d), device="cuda")
    sc = torch.empty((b, hq, L), device="cuda")
    lg = torch.empty((b, hq, L), device="cuda")
    st = torch.zeros((b, hq, 2), device="cuda")
    ctx().attention_gen(q, k, v, out, hkv, L, L, scores=sc, score_stride=L, batch=b, kv_batch_stride=hkv * L * d)
    ctx().attention_gen(q, k, v, out2, hkv, L, L, scores=lg, score_stride=L, batch=b, kv_batch_stride=hkv * L * d,
                        score_stats=st)
    assert torch.equal(out, out2)
    imp, himp = torch.zeros(L, device="cuda"), torch.zeros(hkv * L, device="cuda")
    imp2, himp2 = torch.zeros(L, device="cuda"), torch.zeros(hkv * L, device="cuda")
    ctx().score_reduce(sc, imp, himp, 0.9, b, hq, hkv, L, L, L)
    ctx().score_reduce(lg, imp2, himp2, 0.9, b, hq, hkv, L, L, L, stats=st)
    assert torch.equal(imp, imp2) and torch.equal(himp, himp2)
    i = 5
    _, p = O.attention_gen(host(q[i]), host(k[i]), host(v[i]), hkv, L, L, scores=True, impl="avx2")
    imp1, himp1 = torch.zeros(L, device="cuda"), torch.zeros(hkv * L, device="cuda")
    ctx().score_reduce(lg[i], imp1, himp1, 1.0, 1, hq, hkv, L, L, L, stats=st[i])
    oi, oh = np.zeros(L, np.float32), np.zeros(hkv * L, np.float32)
    O.score_fused_reduce(p, oi, oh, 1.0, 1, hq, hkv, L, L, L)
    check_scores(host(imp1), oi, "importance")
    check_scores(host(himp1), oh, "head importance")


def test_statistics_form_on_the_other_decode_kernels_and_the_fallback_row():
    # vector-ALU kernel (F32 cache), block cache (q4_0), KIVI; and a row without a finite logit,
    # whose uniform weights come out of the statistics as exp(0 - 0) / len.
    import torch
    from blocks_util import random_blocks
    hq, hkv, d, L, cap = 8, 2, 128, 700, 704
    q = normal((1, hq, d), 1)
    k32, v32 = normal((1, hkv, cap, d), 2), normal((1, hkv, cap, d), 3)
    out, sc, out2, lg, st = _decode_both_forms(q, k32, v32, hkv, L, cap, 1)
    assert torch.equal(out, out2)
    assert torch.allclose(torch.exp(lg[..., :L] - st[..., 0:1]) / st[..., 1:2], sc[..., :L], rtol=1e-5, atol=0)
    kq = random_blocks(O.DESC_Q4_0, hkv * cap * d // 32, 5)
    vq = random_blocks(O.DESC_Q4_0, hkv * cap * d // 32, 6)
    import argus_hip as A
    qd, kd, vd = dev(q), dev(kq), dev(vq)
    o1, o2 = torch.empty((1, hq, d), device="cuda"), torch.empty((1, hq, d), device="cuda")
    s1, s2, t2 = torch.zeros((1, hq, cap), device="cuda"), torch.zeros((1, hq, cap), device="cuda"), torch.zeros((1, hq, 2), device="cuda")
    ctx().attention_gen(qd, kd, vd, o1, hkv, L, cap, scores=s1, score_stride=cap, kv_dtype=A.Q4_0)
    ctx().attention_gen(qd, kd, vd, o2, hkv, L, cap, scores=s2, score_stride=cap, kv_dtype=A.Q4_0, score_stats=t2)
    assert torch.equal(o1, o2)
    assert torch.allclose(torch.exp(s2[..., :L] - t2[..., 0:1]) / t2[..., 1:2], s1[..., :L], rtol=1e-5, atol=0)
    # all-NaN query: no finite logit, uniform weights (common.rs:561-577)
    qn = np.full((1, hq, d), np.nan, np.float32)
    out, sc, out2, lg, st = _decode_both_forms(qn, f16(k32), f16(v32), hkv, L, cap, 1)
    assert torch.equal(out, out2)
    assert np.allclose(host(sc)[..., :L], 1.0 / L)
    # the same row over the block cache, in both forms
    qnd = dev(qn)
    ctx().attention_gen(qnd, kd, vd, o1, hkv, L, cap, scores=s1, score_stride=cap, kv_dtype=A.Q4_0)
    ctx().attention_gen(qnd, kd, vd, o2, hkv, L, cap, scores=s2, score_stride=cap, kv_dtype=A.Q4_0, score_stats=t2)
    assert torch.equal(o1, o2) and bool(torch.isfinite(o1).all())
    assert np.allclose(host(s1)[..., :L], 1.0 / L)
    assert np.allclose(host(torch.exp(s2[..., :L] - t2[..., 0:1]) / t2[..., 1:2]), 1.0 / L)
    assert not host(lg)[..., :L].any() and np.array_equal(host(st).reshape(-1, 2), np.tile([0.0, float(L)], (hq, 1)))
    assert ctx().attention_gen(dev(q), dev(f16(k32)), dev(f16(v32)), out, hkv, L, cap, score_stats=st, check=False) == A.ERR_INVALID


@pytest.mark.gpu
def test_config5_batch16_runs_on_the_matrix_core_arm():
    # Two query heads per KV head at head_dim 256: a call that attends 128K rows or more (16 sequences
    # x 4 KV heads x 2048 slots) goes to the matrix-core kernel; below that the vector-ALU kernel is
    # faster and keeps the call.  Same checks as the flow above: outputs, per-position scores (soft
    # cap 50), and the opt-in logits + (max, sum) form against the probability form.
    import torch
    hq, hkv, d, cap, L, batch, softcap = 8, 4, 256, 4096, 2048, 16, 50.0
    q = normal((batch, hq, d), 7)
    kc = np.zeros((batch, hkv, cap, d), np.float16)
    vc = np.zeros((batch, hkv, cap, d), np.float16)
    kc[:, :, :L] = f16(normal((batch, hkv, L, d), 8))
    vc[:, :, :L] = f16(normal((batch, hkv, L, d), 9))
    out, sc, out2, lg, st = _decode_both_forms(q, kc, vc, hkv, L, cap, batch, softcap)
    assert ctx().last_decode_plan()["kernel"] == 1, ctx().last_decode_plan()
    assert torch.equal(out, out2)
    m, l = st[..., 0:1], st[..., 1:2]
    assert torch.allclose(torch.exp(lg[..., :L] - m) / l, sc[..., :L], rtol=1e-5, atol=0)
    got, gsc = host(out), host(sc)
    for b in (0, 7, 15):
        ref, p = O.attention_gen(q[b], kc[b], vc[b], hkv, L, cap, scores=True, scores_stride=cap, softcap=softcap)
        check_attention_out(got[b], ref, "seq %d" % b)
        check_scores(gsc[b, :, :L], p[:, :L], "seq %d" % b)
    # the same shape at 8 sequences stays on the vector-ALU kernel
    out8 = torch.empty((8, hq, d), device="cuda")
    ctx().attention_gen(dev(q[:8]), dev(kc[:8]), dev(vc[:8]), out8, hkv, L, cap, batch=8, kv_batch_stride=hkv * cap * d, softcap=softcap)
    assert ctx().last_decode_plan()["kernel"] == 0, ctx().last_decode_plan()
    for b in (0, 7):
        check_attention_out(host(out8)[b], O.attention_gen(q[b], kc[b], vc[b], hkv, L, cap, softcap=softcap), "seq %d of 8" % b)
