"""Writes tests/golden/*.npz: seeded inputs and the CPU oracle's outputs for each part of the hot path.

The fixtures freeze the oracle: tests/test_golden.py checks that the oracle still reproduces them bit
for bit (CPU) and that the HIP library matches them (GPU), so a change of either shows up against
committed data and not only against the other.  Regenerate with
    python tests/golden/make_golden.py
(the inputs are generated here from fixed seeds; nothing is read from the reference checkout)."""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path[:0] = [os.path.join(HERE, "..", "..", "oracle")]
import oracle as O  # noqa: E402


def save(name, **arrays):
    np.savez_compressed(os.path.join(HERE, name + ".npz"), **arrays)
    print(name, {k: (v.shape, str(v.dtype)) for k, v in arrays.items()})


def main():
    rng = np.random.default_rng(20240607)
    # decode: Backend::attention_gen, F16 HeadMajor cache, scores, plain and soft-capped
    hq, hkv, d, L, cap = 8, 2, 64, 96, 128
    q = rng.standard_normal((hq, d)).astype(np.float32)
    k = rng.standard_normal((hkv, cap, d)).astype(np.float16)
    v = rng.standard_normal((hkv, cap, d)).astype(np.float16)
    out, sc = O.attention_gen(q, k, v, hkv, L, cap, scores=True)
    out_c, sc_c = O.attention_gen(q, k, v, hkv, L, cap, scores=True, softcap=5.0)
    save("decode_f16", q=q, k=k, v=v, dims=np.array([hq, hkv, d, L, cap]), out=out, scores=sc, out_softcap5=out_c,
         scores_softcap5=sc_c)
    # prefill: causal GQA, F32 in/out, chunk offset (cache longer than the chunk)
    hq, hkv, d, S, C, cap = 4, 2, 64, 70, 90, 96
    q = rng.standard_normal((1, S, hq, d)).astype(np.float32)
    k = rng.standard_normal((1, hkv, cap, d)).astype(np.float32)
    v = rng.standard_normal((1, hkv, cap, d)).astype(np.float32)
    out = O.prefill_attention(q, k, v, hkv, C, cap)
    save("prefill_f32", q=q, k=k, v=v, dims=np.array([hq, hkv, d, S, C, cap]), out=out)
    # KIVI: container + fused attention for the three widths
    hq, hkv, d, R, n = 4, 2, 64, 32, 75
    kt = rng.standard_normal((n, hkv, d)).astype(np.float32)
    vt = rng.standard_normal((n, hkv, d)).astype(np.float32)
    kt[:, 0, 3] *= 10.0
    q = rng.standard_normal((hq, d)).astype(np.float32)
    arrays = dict(k_tokens=kt, v_tokens=vt, q=q, dims=np.array([hq, hkv, d, R, n]))
    for bits in (2, 4, 8):
        c = O.kivi_build(kt, vt, R, bits)
        out, sc = O.kivi_attention(q, c, 1.0 / np.sqrt(d), scores=True)
        arrays.update({"qk%d" % bits: c["qk"], "qv%d" % bits: c["qv"], "out%d" % bits: out, "scores%d" % bits: sc})
        arrays["res_k"], arrays["res_v"] = c["res_k"], c["res_v"]
        arrays["q_res_tokens"] = np.array([c["q_tokens"], c["res_tokens"]])
    save("kivi", **arrays)
    # score reduce, PFA side channel, descriptor codec
    n_layers, hq, hkv, L, stride = 3, 8, 2, 50, 64
    scores = rng.random((n_layers, hq, stride)).astype(np.float32)
    imp = rng.random(stride).astype(np.float32)
    himp = rng.random(hkv * stride).astype(np.float32)
    imp2, himp2 = imp.copy(), himp.copy()
    O.score_fused_reduce(scores, imp2, himp2, 0.9, n_layers, hq, hkv, L, stride, stride)
    save("score_reduce", scores=scores, importance_in=imp, head_importance_in=himp, importance_out=imp2,
         head_importance_out=himp2, dims=np.array([n_layers, hq, hkv, L, stride]))
    nq, nkv, d, S, prefix, qs, qw = 6, 2, 32, 9, 40, 31, 4
    q = rng.standard_normal((S, nq, d)).astype(np.float32)
    k = rng.standard_normal(prefix * nkv * d).astype(np.float32)
    summed = np.zeros((nq, prefix), np.float32)
    per_head = np.zeros((qw, nq, prefix), np.float32)
    O.prefill_attention_scores(q, k, nq, nkv, d, S, prefix, nkv * d, d, qs, qw, None, sum_out=summed, per_row=per_head,
                               per_head=True)
    save("pfa", q=q, k=k, dims=np.array([nq, nkv, d, S, prefix, qs, qw]), sum_out=summed, per_head=per_head)
    x = rng.standard_normal(32 * 24).astype(np.float32)
    x[:32] = 0.0
    save("descriptor", x=x, q4_0=O.encode_via_descriptor(O.DESC_Q4_0, x), q2_0=O.encode_via_descriptor(O.DESC_Q2_0, x),
         q4_0_decoded=O.decode_via_descriptor(O.DESC_Q4_0, O.encode_via_descriptor(O.DESC_Q4_0, x), x.size))


def blocks():
    """attention_gen over q4_0 / q8_0 / q2_0 block rows (own generator, so the fixtures above keep their bytes)."""
    rng = np.random.default_rng(20240922)
    hq, hkv, d, L, cap = 8, 2, 64, 80, 96
    q = rng.standard_normal((hq, d)).astype(np.float32)
    arrays = {"q": q, "dims": np.array([hq, hkv, d, L, cap])}
    # q4_0: N(0,1) rows through the reference-shaped encoder
    kq = O.encode_via_descriptor(O.DESC_Q4_0, rng.standard_normal(hkv * cap * d).astype(np.float32))
    vq = O.encode_via_descriptor(O.DESC_Q4_0, rng.standard_normal(hkv * cap * d).astype(np.float32))
    out, sc = O.attention_gen_blocks(q, kq, vq, O.DESC_Q4_0, hkv, L, cap, scores=True)
    arrays.update(k_q4_0=kq, v_q4_0=vq, out_q4_0=out, scores_q4_0=sc)
    # q8_0: random codes, scales sized for unit-variance values (the reference has no q8_0 encoder)
    def q8(n_blocks):
        raw = rng.integers(0, 256, size=(n_blocks, 34), dtype=np.uint8)
        raw[:, 0:2] = rng.uniform(0.005, 0.02, n_blocks).astype(np.float16).view(np.uint8).reshape(n_blocks, 2)
        return raw.reshape(-1)
    k8, v8 = q8(hkv * cap * d // 32), q8(hkv * cap * d // 32)
    out, sc = O.attention_gen_blocks(q, k8, v8, O.DESC_Q8_0, hkv, L, cap, scores=True)
    arrays.update(k_q8_0=k8, v_q8_0=v8, out_q8_0=out, scores_q8_0=sc)
    # q2_0: N(0,1) rows through the reference-shaped asymmetric 2-bit encoder (drawn last: the arrays above keep their bytes)
    k2 = O.encode_via_descriptor(O.DESC_Q2_0, rng.standard_normal(hkv * cap * d).astype(np.float32))
    v2 = O.encode_via_descriptor(O.DESC_Q2_0, rng.standard_normal(hkv * cap * d).astype(np.float32))
    out, sc = O.attention_gen_blocks(q, k2, v2, O.DESC_Q2_0, hkv, L, cap, scores=True)
    arrays.update(k_q2_0=k2, v_q2_0=v2, out_q2_0=out, scores_q2_0=sc)
    save("blocks", **arrays)


if __name__ == "__main__":
    if len(sys.argv) > 1 and sys.argv[1] == "blocks":
        blocks()  # python tests/golden/make_golden.py blocks: only this fixture
    else:
        main()
        blocks()
