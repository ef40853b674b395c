"""GPU parity: attention_gen over block-quantised caches (q4_0 / q4_1 / q8_0) through the C-ABI,
against the oracle's restatement of the reference: each row dequantised exactly as
decode_via_descriptor does, then the scalar F32 attention with its guards
(backend/cpu/common.rs:676-850; `--kv-format` floor kv/standard_format.rs:538-643)."""
import numpy as np
import pytest

import oracle as O
from blocks_util import random_blocks
from gpu_util import ctx, dev, direct_ctx, host, normal, check_attention_out, check_scores

pytestmark = pytest.mark.gpu

FORMATS = {
    "q4_0": (O.DESC_Q4_0, "Q4_0"),
    "q4_1": (O.DESC_Q4_1, "Q4_1"),
    "q8_0": (O.DESC_Q8_0, "Q8_0"),
    "q2_0": (O.DESC_Q2_0, "Q2_0"),
}


def run_case(fmt, hq, hkv, d, L, cap=None, head_major=True, seed=7, scores=True, kv_start=0, encode=False, softcap=0.0, q_gain=1.0,
             score_pad=0, context=None):
    import argus_hip as A
    desc, name = FORMATS[fmt]
    cap = cap or L
    rows = hkv * cap
    if encode:  # real data through the reference's own encoder
        k_raw = O.encode_via_descriptor(desc, normal((rows, d), seed + 1))
        v_raw = O.encode_via_descriptor(desc, normal((rows, d), seed + 2))
    else:
        k_raw = random_blocks(desc, rows * d // 32, seed + 1)
        v_raw = random_blocks(desc, rows * d // 32, seed + 2)
    q = normal((hq, d), seed) * np.float32(q_gain)
    out = dev(np.zeros((hq, d), np.float32))
    sc = dev(np.full((hq, L + score_pad), -7.0, np.float32)) if scores else None
    (context or ctx()).attention_gen(dev(q), dev(k_raw), dev(v_raw), out, hkv, L, cap,
                        layout=A.HEAD_MAJOR if head_major else A.SEQ_MAJOR, scores=sc,
                        score_stride=L + score_pad if scores else 0, kv_start=kv_start, kv_dtype=getattr(A, name), softcap=softcap)
    # oracle: a window that starts at kv_start is the same cache with its first rows cut off
    bb = O.desc_block_bytes(desc)
    row_bytes = d // 32 * bb
    if kv_start:
        assert head_major
        kr = k_raw.reshape(hkv, cap, row_bytes)[:, kv_start:].reshape(-1)
        vr = v_raw.reshape(hkv, cap, row_bytes)[:, kv_start:].reshape(-1)
        ref = O.attention_gen_blocks(q, kr, vr, desc, hkv, L, cap - kv_start, scores=scores, softcap=softcap)
    else:
        ref = O.attention_gen_blocks(q, k_raw, v_raw, desc, hkv, L, cap, head_major=head_major, scores=scores, softcap=softcap)
    what = "%s Hq%d Hkv%d d%d L%d cap%d %s" % (fmt, hq, hkv, d, L, cap, "HM" if head_major else "SM")
    if scores:
        check_attention_out(host(out), ref[0], what)
        got = host(sc)
        check_scores(got[:, :L], ref[1], what)
        assert (got[:, L:] == -7.0).all(), what + ": score row written past its length"
    else:
        check_attention_out(host(out), ref, what)


@pytest.mark.parametrize("L", [509, 510, 511, 512, 1021, 2050, 2051])
def test_score_rows_with_padding_stay_untouched_past_the_length(L):
    # the logits leave in groups of 4 (2 at head_dim 256) tokens per lane; the group that the end of the
    # row cuts is written token by token
    run_case("q4_0", 8, 2, 128, L, score_pad=5, seed=L)
    run_case("q8_0", 14, 2, 64, L, score_pad=3, seed=L + 1)
    run_case("q4_1", 8, 4, 256, L, score_pad=7, seed=L + 2)


@pytest.mark.parametrize("L", [509, 511, 1021, 2051])
def test_scores_stored_inside_the_token_loop(L):
    # the path of chunks too long for the LDS stage, taken at test sizes by a context created under
    # ARGUS_HIP_SCORES=direct
    c = direct_ctx()
    run_case("q4_0", 8, 2, 128, L, score_pad=5, seed=L, context=c)
    assert c.last_decode_plan()["staged_scores"] == 0 and c.last_decode_plan()["kernel"] == 2
    run_case("q8_0", 14, 2, 64, L, score_pad=3, seed=L + 1, context=c)
    run_case("q4_1", 8, 4, 256, L, score_pad=7, seed=L + 2, context=c)
    run_case("q2_0", 12, 1, 128, L, score_pad=1, seed=L + 3, context=c)
    run_case("q4_0", 32, 2, 64, L, score_pad=2, seed=L + 4, context=c)


@pytest.mark.parametrize("fmt", ["q4_0", "q2_0"])
def test_scores_of_groups_wider_than_eight_heads(fmt):
    run_case(fmt, 12, 1, 128, 1531, score_pad=1)
    run_case(fmt, 32, 2, 64, 777, score_pad=2, seed=11)


@pytest.mark.parametrize("fmt", ["q4_0", "q4_1", "q8_0", "q2_0"])
@pytest.mark.parametrize("shape", [(14, 2, 64, 1024), (32, 8, 128, 2048), (8, 4, 256, 1024)])
def test_baseline_shapes(fmt, shape):
    hq, hkv, d, L = shape
    run_case(fmt, hq, hkv, d, L)


def test_blocks_made_by_the_reference_encoder():
    # encode_via_descriptor writes q4_0 and q2_0 (dtype_layout.rs:302-440)
    run_case("q4_0", 32, 8, 128, 4096, encode=True)
    run_case("q4_0", 14, 2, 64, 1024, encode=True, seed=3)
    run_case("q2_0", 32, 8, 128, 4096, encode=True, seed=4)
    run_case("q2_0", 14, 2, 64, 1024, encode=True, seed=5)


@pytest.mark.parametrize("L", [1, 2, 15, 16, 17, 63, 64, 65, 127, 128, 129, 500, 1000])
def test_ragged_lengths(L):
    run_case("q4_0", 8, 2, 128, L, cap=1024, seed=L)
    run_case("q8_0", 4, 4, 64, L, cap=1000 if L <= 1000 else L, seed=L + 1)


@pytest.mark.parametrize("fmt", ["q4_0", "q4_1", "q8_0", "q2_0"])
def test_seq_major_and_window_start(fmt):
    run_case(fmt, 16, 4, 128, 777, cap=800, head_major=False, seed=11)
    run_case(fmt, 16, 4, 128, 300, cap=800, kv_start=411, seed=12)


def test_group_of_sixteen_and_single_head():
    run_case("q4_0", 32, 2, 64, 512, seed=21)
    run_case("q4_0", 1, 1, 128, 512, seed=22)


def test_long_row_at_32k_tokens():
    run_case("q4_0", 32, 8, 128, 32768, scores=True, seed=5)


@pytest.mark.parametrize("fmt,hq,hkv,d,L", [("q4_1", 8, 4, 256, 20000), ("q4_0", 14, 2, 64, 20000), ("q8_0", 8, 2, 256, 20000),
                                            ("q4_1", 14, 2, 64, 33000), ("q8_0", 4, 4, 64, 17001), ("q4_0", 16, 2, 256, 9999),
                                            ("q2_0", 14, 2, 64, 20000), ("q2_0", 32, 8, 128, 20000), ("q2_0", 16, 8, 256, 9999)])
def test_several_tiles_per_wave_at_every_head_dim(fmt, hq, hkv, d, L):
    # Long rows give every wave more than one tile, so the tile requested ahead of the one being
    # worked on is the one consumed next (head_dim 64 pairs two tiles per request, 256 splits one over two).
    run_case(fmt, hq, hkv, d, L, cap=L + 3, seed=L % 97)


@pytest.mark.parametrize("fmt", ["q4_0", "q4_1", "q8_0", "q2_0"])
@pytest.mark.parametrize("d", [64, 128, 256])
def test_ragged_lengths_at_every_head_dim(fmt, d):
    for L in (1, 7, 16, 17, 31, 32, 33, 47, 48, 49, 64, 65, 100, 129, 333):
        run_case(fmt, 8, 2, d, L, cap=400, seed=L + d)


@pytest.mark.parametrize("fmt", ["q4_0", "q4_1", "q8_0", "q2_0"])
@pytest.mark.parametrize("d", [64, 128, 256])
def test_every_group_width_with_and_without_scores(fmt, d):
    # Up to four query heads per KV head the kernel keeps one head per lane group (the logits MFMA
    # has the tokens in its columns), five to eight at head_dim 64 and 128 two heads per lane group;
    # wider groups keep the heads in the columns.  Every head must get its own logits in each, with
    # the scores emitted or not, over ragged and multi-tile rows.
    for g in (1, 2, 3, 4, 5, 6, 7, 8) + ((9, 16) if d != 256 else ()):  # (head_dim 256 takes groups of up to 8)
        for L in (97, 1300):
            run_case(fmt, 2 * g, 2, d, L, cap=L + 5, seed=g + L + d, scores=bool((g + L) & 1))
            run_case(fmt, 2 * g, 2, d, L, cap=L + 5, seed=g + L + d + 1, scores=not ((g + L) & 1))


@pytest.mark.parametrize("fmt", ["q4_0", "q4_1", "q8_0", "q2_0"])
@pytest.mark.parametrize("hq,hkv,d", [(8, 2, 64), (14, 2, 64), (32, 8, 128), (16, 2, 128), (8, 4, 256)])
def test_value_scales_from_tiny_to_large(fmt, hq, hkv, d):
    # Groups of up to four heads carry a V block's scale on the attention weights instead of on its
    # codes (the product of a weight and a scale is rounded to f16 before the matrix multiply), wider
    # groups scale the codes: V scales (and minima) spread over 2^-12 .. 2^4 times the usual ones
    # pin both against the oracle, relative to the largest output.
    import argus_hip as A
    desc, name = FORMATS[fmt]
    L = 1500
    rows = hkv * L
    bb = O.desc_block_bytes(desc)
    k_raw = random_blocks(desc, rows * d // 32, 31)
    v_raw = random_blocks(desc, rows * d // 32, 32).reshape(-1, bb).copy()
    gain = np.exp2(np.random.default_rng(33).integers(-12, 5, size=v_raw.shape[0])).astype(np.float32)
    hdr = v_raw[:, :4].copy().view(np.float16).astype(np.float32)  # (d, m or the first code bytes)
    n_hdr = 2 if desc[2] == O.SCALE_F16_MIN else 1
    scaled = (hdr[:, :n_hdr] * gain[:, None]).astype(np.float16)
    v_raw[:, :2 * n_hdr] = scaled.view(np.uint8).reshape(-1, 2 * n_hdr)
    v_raw = v_raw.reshape(-1)
    q = normal((hq, d), 30)
    out = dev(np.zeros((hq, d), np.float32))
    ctx().attention_gen(dev(q), dev(k_raw), dev(v_raw), out, hkv, L, L, kv_dtype=getattr(A, name))
    ref = O.attention_gen_blocks(q, k_raw, v_raw, desc, hkv, L, L)
    got = host(out)
    assert np.all(np.isfinite(got))
    err = np.abs(got.astype(np.float64) - ref) / np.abs(ref).max()
    assert err.max() <= 2e-3 and err.mean() <= 1e-3, "%s Hq%d Hkv%d d%d: max %g mean %g of the largest output" % (fmt, hq, hkv, d, err.max(), err.mean())


@pytest.mark.parametrize("fmt,hq,hkv,d,L", [("q4_0", 16, 8, 256, 2048), ("q8_0", 8, 4, 256, 1000), ("q4_1", 32, 8, 128, 1500), ("q4_0", 14, 2, 64, 777),
                                            ("q2_0", 32, 8, 128, 900)])
def test_soft_cap_on_block_caches(fmt, hq, hkv, d, L):
    # Gemma-2 style logit soft-cap (cap * tanh(logit / cap)) with queries large enough that the cap bites.
    run_case(fmt, hq, hkv, d, L, cap=L + 8, seed=L % 89, softcap=50.0, q_gain=4.0)
    run_case(fmt, hq, hkv, d, L, cap=L + 8, seed=L % 89 + 1, softcap=3.0)


@pytest.mark.parametrize("fmt", ["q4_0", "q4_1", "q8_0", "q2_0"])
@pytest.mark.parametrize("hq,hkv,d,L,cap", [(14, 2, 64, 700, 1500), (32, 8, 128, 1000, 4096), (8, 4, 256, 333, 800), (8, 2, 128, 9000, 20000),
                                            (16, 2, 128, 700, 1500), (14, 2, 128, 2100, 2500)])
def test_index_list_over_block_caches(fmt, hq, hkv, d, L, cap):
    # Post-eviction addressing: token t lives in slot kv_index[t] (any order, here shuffled), and the
    # result is the attention over the gathered rows.
    import argus_hip as A
    desc, name = FORMATS[fmt]
    k_raw = random_blocks(desc, hkv * cap * d // 32, L + 1)
    v_raw = random_blocks(desc, hkv * cap * d // 32, L + 2)
    q = normal((hq, d), L)
    idx = np.random.default_rng(L + d).choice(cap, L, replace=False).astype(np.int32)
    out = dev(np.zeros((hq, d), np.float32))
    sc = dev(np.zeros((hq, L), np.float32))
    ctx().attention_gen(dev(q), dev(k_raw), dev(v_raw), out, hkv, L, cap, scores=sc, score_stride=L,
                        kv_index=dev(idx), kv_dtype=getattr(A, name))
    ref = O.attention_gen_blocks(q, k_raw, v_raw, desc, hkv, L, cap, scores=True, kv_index=idx)
    what = "%s indexed Hq%d Hkv%d d%d L%d cap%d" % (fmt, hq, hkv, d, L, cap)
    check_attention_out(host(out), ref[0], what)
    check_scores(host(sc), ref[1], what)


def test_index_list_batch_and_fallback():
    import argus_hip as A
    desc, _ = FORMATS["q4_0"]
    b, hq, hkv, d, L, cap = 3, 8, 2, 64, 500, 640
    raws = [(random_blocks(desc, hkv * cap * d // 32, 50 + i), random_blocks(desc, hkv * cap * d // 32, 60 + i)) for i in range(b)]
    q = normal((b, hq, d), 9)
    q[1, 2, 0] = np.nan  # one head of one sequence: uniform weights over the indexed rows
    idx = np.stack([np.random.default_rng(70 + i).choice(cap, L, replace=False) for i in range(b)]).astype(np.int32)
    out = dev(np.zeros((b, hq, d), np.float32))
    ctx().attention_gen(dev(q), dev(np.stack([r[0] for r in raws])), dev(np.stack([r[1] for r in raws])), out, hkv, L, cap,
                        batch=b, kv_batch_stride=hkv * cap * d, kv_index=dev(idx), index_batch_stride=L, kv_dtype=A.Q4_0)
    got = host(out)
    for i in range(b):
        ref = O.attention_gen_blocks(q[i], raws[i][0], raws[i][1], desc, hkv, L, cap, kv_index=idx[i])
        for h in range(hq):
            if i == 1 and h == 2:
                np.testing.assert_allclose(got[i, h], ref[h], atol=2e-5)
            else:
                check_attention_out(got[i, h], ref[h], "seq %d head %d" % (i, h))


def test_batch_of_sequences():
    import argus_hip as A
    desc, _ = FORMATS["q4_0"]
    b, hq, hkv, d, L, cap = 3, 8, 2, 128, 700, 768
    raws = [(random_blocks(desc, hkv * cap * d // 32, 30 + i), random_blocks(desc, hkv * cap * d // 32, 40 + i)) for i in range(b)]
    q = normal((b, hq, d), 9)
    k = dev(np.stack([r[0] for r in raws]))
    v = dev(np.stack([r[1] for r in raws]))
    out = dev(np.zeros((b, hq, d), np.float32))
    sc = dev(np.zeros((b, hq, L), np.float32))
    ctx().attention_gen(dev(q), k, v, out, hkv, L, cap, scores=sc, score_stride=L, batch=b,
                        kv_batch_stride=hkv * cap * d, kv_dtype=A.Q4_0)
    for i in range(b):
        ref = O.attention_gen_blocks(q[i], raws[i][0], raws[i][1], desc, hkv, L, cap, scores=True)
        check_attention_out(host(out)[i], ref[0], "seq %d" % i)
        check_scores(host(sc)[i], ref[1], "seq %d" % i)


def test_nan_query_takes_the_uniform_fallback():
    # A NaN query makes every logit NaN -> -inf -> uniform weights (common.rs:790-813).
    import argus_hip as A
    desc, _ = FORMATS["q4_0"]
    hq, hkv, d, L = 4, 2, 64, 200
    k_raw = random_blocks(desc, hkv * L * d // 32, 1)
    v_raw = random_blocks(desc, hkv * L * d // 32, 2)
    q = normal((hq, d), 3)
    q[1, 5] = np.nan
    out = dev(np.zeros((hq, d), np.float32))
    sc = dev(np.zeros((hq, L), np.float32))
    ctx().attention_gen(dev(q), dev(k_raw), dev(v_raw), out, hkv, L, L, scores=sc, score_stride=L, kv_dtype=A.Q4_0)
    ref = O.attention_gen_blocks(q, k_raw, v_raw, desc, hkv, L, L, scores=True)
    got, gsc = host(out), host(sc)
    np.testing.assert_allclose(gsc[1], 1.0 / L, rtol=1e-6)
    np.testing.assert_allclose(got[1], ref[0][1], atol=2e-5)
    for h in (0, 2, 3):
        check_attention_out(got[h], ref[0][h], "head %d" % h)


def test_unsupported_combinations_are_refused():
    import argus_hip as A
    desc, _ = FORMATS["q4_0"]
    hq, hkv, d, L = 4, 2, 64, 64
    k = dev(random_blocks(desc, hkv * L * d // 32, 1))
    q = dev(normal((hq, d), 3))
    out = dev(np.zeros((hq, d), np.float32))
    c = ctx()
    q17 = dev(normal((34, d), 3))
    out17 = dev(np.zeros((34, d), np.float32))
    assert c.attention_gen(q17, k, k, out17, 2, L, L, kv_dtype=A.Q4_0, check=False) == A.ERR_UNSUPPORTED
