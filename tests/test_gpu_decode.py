"""GPU parity: argus_hip_attention_gen (through the C ABI) against the CPU oracle."""
import numpy as np
import pytest

import oracle as O
import textbook as T
from gpu_util import check_attention_out, check_scores, ctx, dev, direct_ctx, host, normal

pytestmark = pytest.mark.gpu


def run_decode(q, k, v, hkv, L, capacity, layout=0, scores=False, score_stride=None, context=None, **kw):
    import torch
    import argus_hip as A
    qd, kd, vd = dev(q), dev(k), dev(v)
    out = torch.full(q.shape, float("nan"), dtype=torch.float32, device="cuda")
    sc = None
    stride = 0
    if scores:
        stride = score_stride or L
        sc = torch.full(q.shape[:-1] + (stride,), -7.0, dtype=torch.float32, device="cuda")
    (context or ctx()).attention_gen(qd, kd, vd, out, hkv, L, capacity, layout=layout, scores=sc,
                                     score_stride=stride, **kw)
    return (host(out), host(sc)) if scores else host(out)


def f16(x):
    return O.f32_to_f16_bits(x).view(np.float16)


@pytest.mark.parametrize("kv", ["f32", "f16"])
def test_reference_unit_case(kv):
    # engine/src/backend/cpu/x86.rs:1811-1973 inputs (LCG seeds 42/137/53), its own tolerances.
    hq, hkv, d, L, cap = 4, 2, 64, 16, 32
    q = O.gen_data(hq * d, 42).reshape(hq, d)
    k = O.gen_data(hkv * cap * d, 137).reshape(hkv, cap, d)
    v = O.gen_data(hkv * cap * d, 53).reshape(hkv, cap, d)
    if kv == "f16":
        k, v = f16(k), f16(v)
    got = run_decode(q, k, v, hkv, L, cap)
    ref = O.attention_gen(q, k, v, hkv, L, cap)
    assert np.abs(got - ref).max() < (1e-4 if kv == "f32" else 1e-3)
    check_attention_out(got, O.attention_gen(q, k, v, hkv, L, cap, impl="avx2"))


# engine/tests/test_attention_flash_decoding.rs:260-651 matrix: GQA ratios, chunk boundaries.
MATRIX = [
    (4, 4, 64, 1), (4, 4, 64, 32), (4, 2, 64, 33), (8, 2, 64, 256), (8, 2, 64, 1023),
    (8, 2, 64, 1024), (8, 2, 64, 1025), (12, 2, 128, 2047), (12, 2, 128, 2500),
    (8, 2, 128, 4096), (14, 2, 64, 1024), (8, 4, 256, 777), (32, 8, 128, 300), (6, 2, 256, 129),
    (16, 2, 64, 555), (3, 1, 128, 70), (5, 1, 64, 200),
    # GQA groups wider than 8 (12, 16): F32 caches and short rows take several head tiles per KV head
    (24, 2, 128, 63), (32, 2, 64, 100), (96, 8, 64, 300), (12, 1, 256, 40),
]


@pytest.mark.parametrize("hq,hkv,d,L", MATRIX)
@pytest.mark.parametrize("kv", ["f16", "f32"])
def test_decode_matrix(hq, hkv, d, L, kv):
    cap = L + 19
    q = normal((hq, d), 42 + L)
    k = normal((hkv, cap, d), 137 + L)
    v = normal((hkv, cap, d), 53 + L)
    if kv == "f16":
        k, v = f16(k), f16(v)
    got, sc = run_decode(q, k, v, hkv, L, cap, scores=True, score_stride=cap, context=direct_ctx())
    assert direct_ctx().last_decode_plan()["staged_scores"] == 0, "logits were staged in LDS after all"
    ref, p = O.attention_gen(q, k, v, hkv, L, cap, scores=True, scores_stride=cap)
    check_attention_out(got, ref, "out")
    check_scores(sc[:, :L], p[:, :L], "scores")
    assert np.all(sc[:, L:] == -7.0), "score columns beyond cache_seq_len must stay untouched"
    assert np.abs(sc[:, :L].sum(axis=1) - 1.0).max() < 1e-3
    # independent f64 check as well
    r64, p64 = T.decode_attention(q, k, v, hkv, L)
    check_attention_out(got, r64, "out vs f64")
    # no-scores launch (single-split direct path for short L) gives the same output
    # (another cut of the row: the probabilities are rounded to f16 against another running maximum)
    got2 = run_decode(q, k, v, hkv, L, cap)
    assert np.abs(got2 - got).max() < 1e-4
    check_attention_out(got2, r64, "no-scores out vs f64")


def test_seq_major_layout():
    hq, hkv, d, L = 8, 2, 128, 700
    q = normal((hq, d), 1)
    k = f16(normal((L, hkv, d), 2))
    v = f16(normal((L, hkv, d), 3))
    got = run_decode(q, k, v, hkv, L, 0, layout=1)
    ref = O.attention_gen(q, k, v, hkv, L, 0, head_major=False)
    check_attention_out(got, ref)


def test_closed_form_zero_keys():
    # engine/src/kv/standard_format.rs:3095-3199: K = 0 => uniform; out = mean(V), scores 0.5/0.5.
    hq, hkv, d = 2, 1, 64
    q = normal((hq, d), 5)
    k = np.zeros((hkv, 4, d), np.float16)
    v = np.zeros((hkv, 4, d), np.float16)
    v[0, 0], v[0, 1] = 1.0, 3.0
    got, sc = run_decode(q, k, v, hkv, 2, 4, scores=True)
    assert np.allclose(got, 2.0, atol=1e-6) and np.allclose(sc, 0.5, atol=1e-7)
    assert np.allclose(run_decode(q, k, v, hkv, 1, 4), 1.0, atol=1e-7)


@pytest.mark.parametrize("L", [8, 3000])
def test_nan_guards(L):
    # engine/src/backend/cpu/common.rs:555-584.
    hq, hkv, d = 4, 2, 64
    q = normal((hq, d), 9)
    k = normal((hkv, L, d), 10)
    v = normal((hkv, L, d), 11)
    k[0, 3, 0] = np.nan
    k[1, L - 1, 5] = np.nan
    got, sc = run_decode(q, k, v, hkv, L, L, scores=True)
    ref, p = O.attention_gen(q, k, v, hkv, L, L, scores=True)
    check_attention_out(got, ref)
    check_scores(sc, p)
    assert sc[0, 3] == 0.0 and sc[3, L - 1] == 0.0
    # every logit NaN for kv head 0 -> uniform weights, out = mean of V rows
    k[0] = np.nan
    got, sc = run_decode(q, k, v, hkv, L, L, scores=True)
    ref, p = O.attention_gen(q, k, v, hkv, L, L, scores=True)
    check_attention_out(got, ref)
    check_scores(sc, p)
    assert np.allclose(sc[0], 1.0 / L)
    got2 = run_decode(q, k, v, hkv, L, L)
    check_attention_out(got2, ref)


def test_softcap_index_and_window_start():
    hq, hkv, d, L, cap = 8, 4, 256, 2048, 4096
    q = normal((hq, d), 21) * 3.0
    k = f16(normal((hkv, cap, d), 22))
    v = f16(normal((hkv, cap, d), 23))
    got, sc = run_decode(q, k, v, hkv, L, cap, scores=True, softcap=5.0)
    ref, p = O.attention_gen(q, k, v, hkv, L, cap, scores=True, softcap=5.0)
    check_attention_out(got, ref)
    check_scores(sc, p)
    r64, p64 = T.decode_attention(q, k, v, hkv, L, softcap=5.0)
    check_attention_out(got, r64)
    # index list == attention over the gathered rows
    idx = np.sort(np.random.default_rng(3).choice(cap, L, replace=False)).astype(np.int32)
    got = run_decode(q, k, v, hkv, L, cap, kv_index=dev(idx))
    ref = O.attention_gen(q, k, v, hkv, L, cap, kv_index=idx)
    check_attention_out(got, ref)
    # kv_start: attends slots [kv_start, kv_start + L)
    got = run_decode(q, k, v, hkv, 1000, cap, kv_start=77)
    ref = O.attention_gen(q, np.ascontiguousarray(k[:, 77:1077]), np.ascontiguousarray(v[:, 77:1077]), hkv, 1000, 1000)
    check_attention_out(got, ref)


@pytest.mark.parametrize("L", [2, 33, 65])
def test_scores_of_a_short_row_are_normalised_by_the_unrounded_sum(L):
    # The matrix cores consume f16-rounded weights; the scores are exp / sum(exp) in f32.  Over a few
    # dozen tokens a sum of the rounded weights differs from the f32 sum by up to 2^-12 and moved every
    # score of a head past the 1e-4 bar (Hq48 Hkv8 d128 L65, soft-cap 30: 1.07e-4 on two heads).
    # Inputs follow that draw: generator 1100269, Q doubled, window starting at slot 1 of capacity L+6.
    hq, hkv, d, cap, start = 48, 8, 128, L + 6, 1
    rng = np.random.default_rng(1100269)
    shape = [int(rng.choice([64, 128, 256])), int(rng.choice([1, 2, 3, 4, 8])), int(rng.choice([1, 2, 3, 4, 6, 7, 8, 12, 16])),
             int(rng.choice([1, 3, 17, 63, 64, 65, 100, 257, 700, 1500, 4097, 9000, 20000]))]
    assert shape == [128, 8, 6, 65]  # the draws that picked the shape, so that Q, K and V are that case's
    rng.integers(0, 50), rng.choice(["f16", "f32", "q4_0", "q4_1", "q8_0", "q2_0"]), rng.integers(0, 2)
    rng.choice([0.0, 0.0, 7.0, 30.0]), rng.integers(0, 3), rng.integers(0, 7), rng.integers(0, 4)
    q = rng.standard_normal((hq, d)).astype(np.float32) * np.float32(2.0)
    k = f16(rng.standard_normal((hkv, cap, d)).astype(np.float32))
    v = f16(rng.standard_normal((hkv, cap, d)).astype(np.float32))
    for softcap in (30.0, 0.0):
        got, sc = run_decode(q, k, v, hkv, L, cap, scores=True, softcap=softcap, kv_start=start)
        ref, p = O.attention_gen(q, np.ascontiguousarray(k[:, start:]), np.ascontiguousarray(v[:, start:]), hkv, L,
                                 cap - start, scores=True, softcap=softcap)
        check_attention_out(got, ref)
        check_scores(sc, p)
        assert np.abs(sc.sum(axis=1) - 1.0).max() < 1e-5


@pytest.mark.parametrize("hq,hkv,d,L,cap", [(32, 8, 128, 1500, 1536), (14, 2, 64, 777, 800)])
def test_softcap_on_the_matrix_core_path(hq, hkv, d, L, cap):
    # F16 KV, no index list, d in {64, 128}: soft-capped logits run through the MFMA kernel; same
    # definition (cap * tanh(logit / cap)), emitted scores included; a NaN key still counts as -inf.
    q = normal((hq, d), 61) * 2.0
    k = f16(normal((hkv, cap, d), 62))
    v = f16(normal((hkv, cap, d), 63))
    for softcap in (5.0, 50.0):
        got, sc = run_decode(q, k, v, hkv, L, cap, scores=True, softcap=softcap)
        ref, p = O.attention_gen(q, k, v, hkv, L, cap, scores=True, softcap=softcap)
        check_attention_out(got, ref)
        check_scores(sc, p)
        r64, p64 = T.decode_attention(q, k, v, hkv, L, softcap=softcap)
        check_attention_out(got, r64)
    k2 = k.copy()
    k2[0, 5, 3] = np.float16(np.nan)
    got, sc = run_decode(q, k2, v, hkv, L, cap, scores=True, softcap=5.0)
    ref, p = O.attention_gen(q, k2, v, hkv, L, cap, scores=True, softcap=5.0)
    check_attention_out(got, ref)
    check_scores(sc, p)
    assert (sc[:hq // hkv, 5] == 0).all()


def test_batched_sequences_match_looped_calls():
    # the reference has no batch dimension (engine/src/backend.rs:277-295): batch == a loop.
    b, hq, hkv, d, L, cap = 5, 32, 8, 128, 1500, 1536
    q = normal((b, hq, d), 42)
    k = f16(normal((b, hkv, cap, d), 137))
    v = f16(normal((b, hkv, cap, d), 53))
    got, sc = run_decode(q, k, v, hkv, L, cap, scores=True, batch=b, kv_batch_stride=hkv * cap * d)
    for i in range(b):
        ref, p = O.attention_gen(q[i], k[i], v[i], hkv, L, cap, scores=True)
        check_attention_out(got[i], ref, "seq %d" % i)
        check_scores(sc[i], p, "seq %d" % i)


@pytest.mark.parametrize("hq,hkv,d,L", [(32, 8, 128, 4096), (14, 2, 64, 1024), (16, 1, 64, 3000), (3, 3, 128, 777),
                                       (32, 4, 256, 8192), (24, 6, 256, 9000), (7, 1, 128, 20000)])
def test_calls_without_scores_alternating_lengths(hq, hkv, d, L):
    # Calls of different lengths (so different split counts) alternate on one context and share its
    # partial workspace: state left over from the previous call would show as a wrong output.
    cap = L + 5
    q = normal((hq, d), 1 + L)
    k = f16(normal((hkv, cap, d), 2 + L))
    v = f16(normal((hkv, cap, d), 3 + L))
    lengths = [L, 64 + L // 3, L, 100]
    refs = {n: O.attention_gen(q, k, v, hkv, n, cap) for n in set(lengths)}
    for rep in range(3):
        for n in lengths:
            check_attention_out(run_decode(q, k, v, hkv, n, cap), refs[n], "len %d rep %d" % (n, rep))


def test_calls_without_scores_batch_and_fallback():
    b, hq, hkv, d, L, cap = 6, 16, 4, 128, 2000, 2048
    q = normal((b, hq, d), 5)
    k = f16(normal((b, hkv, cap, d), 6))
    v = f16(normal((b, hkv, cap, d), 7))
    k[2, 1] = np.nan  # every logit of that KV head's four query heads is NaN: uniform weights
    k[4, 3, 17, 0] = np.nan
    for rep in range(2):
        got = run_decode(q, k, v, hkv, L, cap, batch=b, kv_batch_stride=hkv * cap * d)
        for i in range(b):
            check_attention_out(got[i], O.attention_gen(q[i], k[i], v[i], hkv, L, cap), "seq %d rep %d" % (i, rep))


@pytest.mark.parametrize("hq,hkv,d,L,cap", [(32, 8, 128, 3000, 8192), (14, 2, 64, 1000, 1024), (8, 2, 128, 20000, 40000),
                                           (32, 4, 256, 9000, 12000), (5, 1, 64, 77, 300)])
def test_index_list_on_the_matrix_core_path(hq, hkv, d, L, cap):
    # Post-eviction addressing on F16 caches: token t lives in slot kv_index[t] (shuffled here), the
    # result is the attention over the gathered rows; with scores, without, and with a soft-cap.
    q = normal((hq, d), L)
    k = f16(normal((hkv, cap, d), L + 1))
    v = f16(normal((hkv, cap, d), L + 2))
    idx = np.random.default_rng(L).choice(cap, L, replace=False).astype(np.int32)
    got, sc = run_decode(q, k, v, hkv, L, cap, scores=True, kv_index=dev(idx))
    ref, p = O.attention_gen(q, k, v, hkv, L, cap, scores=True, kv_index=idx)
    check_attention_out(got, ref, "indexed")
    check_scores(sc, p, "indexed")
    check_attention_out(run_decode(q, k, v, hkv, L, cap, kv_index=dev(idx)), ref, "indexed, no scores")
    got = run_decode(q * 3.0, k, v, hkv, L, cap, kv_index=dev(idx), softcap=8.0)
    check_attention_out(got, O.attention_gen(q * 3.0, k, v, hkv, L, cap, kv_index=idx, softcap=8.0), "indexed + soft-cap")


def test_index_list_per_sequence_in_a_batch():
    b, hq, hkv, d, L, cap = 4, 16, 4, 128, 1500, 2048
    q = normal((b, hq, d), 1)
    k = f16(normal((b, hkv, cap, d), 2))
    v = f16(normal((b, hkv, cap, d), 3))
    idx = np.stack([np.random.default_rng(10 + i).choice(cap, L, replace=False) for i in range(b)]).astype(np.int32)
    got = run_decode(q, k, v, hkv, L, cap, batch=b, kv_batch_stride=hkv * cap * d, kv_index=dev(idx), index_batch_stride=L)
    for i in range(b):
        check_attention_out(got[i], O.attention_gen(q[i], k[i], v[i], hkv, L, cap, kv_index=idx[i]), "seq %d" % i)


def test_config1_qwen_shape():
    # benchmark configuration 1: Hq14 Hkv2 d64 L1024, f32 N(0,1) -> F16 KV, scale 1/8.
    hq, hkv, d, L = 14, 2, 64, 1024
    q = normal((hq, d), 42)
    k = f16(normal((hkv, L, d), 137))
    v = f16(normal((hkv, L, d), 53))
    got = run_decode(q, k, v, hkv, L, L)
    check_attention_out(got, O.attention_gen(q, k, v, hkv, L, L))
    check_attention_out(got, O.attention_gen(q, k, v, hkv, L, L, impl="avx2"))
    got_cap = run_decode(q, np.concatenate([k, k], 1), np.concatenate([v, v], 1), hkv, L, 2 * L)
    assert np.array_equal(got, got_cap)


@pytest.mark.parametrize("L", [4096, 32768])
def test_config3_llama8b_shape_single_sequence(L):
    hq, hkv, d = 32, 8, 128
    q = normal((hq, d), 42)
    k = f16(normal((hkv, L, d), 137))
    v = f16(normal((hkv, L, d), 53))
    got, sc = run_decode(q, k, v, hkv, L, L, scores=True)
    ref, p = O.attention_gen(q, k, v, hkv, L, L, scores=True, impl="avx2")
    check_attention_out(got, ref)
    check_scores(sc, p)


def test_config3_batch16_at_32k_properties_and_sampled_parity():
    # 2 GiB of KV: generated on the device; parity on two sampled sequences, plus
    # size-independent properties on all of them.
    import torch
    b, hq, hkv, d, L = 16, 32, 8, 128, 32768
    g = torch.Generator(device="cuda").manual_seed(137)
    k = torch.randn((b, hkv, L, d), generator=g, device="cuda", dtype=torch.float32).half()
    v = torch.randn((b, hkv, L, d), generator=g, device="cuda", dtype=torch.float32).half()
    q = dev(normal((b, hq, d), 42))
    out = torch.empty((b, hq, d), dtype=torch.float32, device="cuda")
    sc = torch.empty((b, hq, L), dtype=torch.float32, device="cuda")
    ctx().attention_gen(q, k, v, out, hkv, L, L, scores=sc, score_stride=L, batch=b,
                        kv_batch_stride=hkv * L * d)
    torch.cuda.synchronize()
    # probabilities: rows sum to 1, out == P @ V (linearity), permutation of tokens is a no-op.
    assert (sc.sum(-1) - 1).abs().max().item() < 1e-3
    pv = torch.einsum("bgrl,bgld->bgrd", sc.view(b, hkv, hq // hkv, L), v.float()).reshape(b, hq, d)
    assert (pv - out).abs().max().item() < 1e-4
    for i in (0, 11):
        ref = O.attention_gen(host(q[i]), host(k[i]), host(v[i]), hkv, L, L, impl="avx2")
        check_attention_out(host(out[i]), ref, "seq %d" % i)
    # The weights enter the matrix cores rounded to f16 relative to the running maximum, so the
    # token order changes the rounding: measured 7e-6 .. 9e-6 over a dozen permutations (outputs
    # up to 3e-2), two orders below the 2e-3 parity bar.  Seeded, so the case is reproducible.
    perm = torch.randperm(L, device="cuda", generator=torch.Generator(device="cuda").manual_seed(5))
    out2 = torch.empty_like(out[:1])
    ctx().attention_gen(q[:1], k[0][:, perm].contiguous(), v[0][:, perm].contiguous(), out2, hkv, L, L)
    assert (out2[0] - out[0]).abs().max().item() < 3e-5


def test_config3_batch16_at_4k():
    # benchmark configuration 3 at its shorter length: 16 independent sequences of 4096 tokens in one launch,
    # every one checked against the oracle, with and without scores.
    b, hq, hkv, d, L = 16, 32, 8, 128, 4096
    q = normal((b, hq, d), 42)
    k = f16(normal((b, hkv, L, d), 137))
    v = f16(normal((b, hkv, L, d), 53))
    got, sc = run_decode(q, k, v, hkv, L, L, scores=True, batch=b, kv_batch_stride=hkv * L * d)
    plain = run_decode(q, k, v, hkv, L, L, batch=b, kv_batch_stride=hkv * L * d)
    for i in range(b):
        ref, p = O.attention_gen(q[i], k[i], v[i], hkv, L, L, scores=True, impl="avx2")
        check_attention_out(got[i], ref, "seq %d" % i)
        check_attention_out(plain[i], ref, "seq %d, no scores" % i)
        check_scores(sc[i], p, "seq %d" % i)


def test_index_list_with_slots_at_and_beyond_the_capacity():
    # Slots near capacity-1 are ordinary; an entry outside [0, capacity) must never steer a load out
    # of the cache (the attended row for it is unspecified, so only the in-range lists are compared).
    # Short rows, F32 caches and block formats read rows with plain loads, F16 rows through a bounded
    # buffer descriptor: both kinds are covered.  The caches sit at the end of their allocations.
    import argus_hip as A
    hq, hkv, d, cap = 8, 2, 128, 96
    for L, kind in ((40, "f16"), (80, "f16"), (40, "f32"), (80, "f32")):
        q = normal((hq, d), L)
        k, v = normal((hkv, cap, d), L + 1), normal((hkv, cap, d), L + 2)
        if kind == "f16":
            k, v = f16(k), f16(v)
        idx = (cap - 1 - np.arange(L)).astype(np.int32)  # cap-1, cap-2, ...
        got = run_decode(q, k, v, hkv, L, cap, kv_index=dev(idx))
        check_attention_out(got, O.attention_gen(q, k, v, hkv, L, cap, kv_index=idx), "%s L%d" % (kind, L))
        bad = idx.copy()
        bad[3], bad[7] = cap + 5000000, -3
        out = run_decode(q, k, v, hkv, L, cap, kv_index=dev(bad))
        assert np.all(np.isfinite(out)), "%s L%d: stale slots" % (kind, L)
    q = dev(normal((hq, d), 1))
    kd = dev(f16(normal((hkv, cap, d), 2)))
    out = dev(np.zeros((hq, d), np.float32))
    ix = dev(np.arange(40, dtype=np.int32))
    assert ctx().attention_gen(q, kd, kd, out, hkv, 40, 0, kv_index=ix, check=False) == A.ERR_INVALID
    assert "capacity" in ctx().last_error()


def test_head_dim_outside_the_kernels_is_refused_for_every_cache_type():
    # return codes only: nothing is launched
    import torch
    import argus_hip as A
    c = ctx()
    for d in (32, 80, 96, 512):
        q = torch.zeros((4, d), device="cuda")
        out = torch.zeros((4, d), device="cuda")
        kf = torch.zeros((2, 8, d), device="cuda", dtype=torch.float16)
        assert c.attention_gen(q, kf, kf, out, 2, 8, 8, check=False) == A.ERR_UNSUPPORTED, d
        assert c.attention_gen(q, kf.float(), kf.float(), out, 2, 8, 8, check=False) == A.ERR_UNSUPPORTED, d
        if d % 32 == 0:
            for kvt, bb in ((A.Q4_0, 18), (A.Q4_1, 20), (A.Q8_0, 34), (A.Q2_0, 12)):
                blk = torch.zeros(2 * 8 * (d // 32) * bb + 64, device="cuda", dtype=torch.uint8)
                assert c.attention_gen(q, blk, blk, out, 2, 8, 8, kv_dtype=kvt, check=False) == A.ERR_UNSUPPORTED, (d, kvt)
                assert "head_dim" in c.last_error()
    q = torch.zeros((4, 128), device="cuda")
    blk = torch.zeros(1 << 16, device="cuda", dtype=torch.uint8)
    assert c.attention_gen(q, blk, blk, q.clone(), 2, 8, 8, kv_dtype=9, check=False) == A.ERR_UNSUPPORTED


def test_argument_errors_return_negative_codes():
    import torch
    import argus_hip as A
    q = torch.zeros((4, 64), device="cuda")
    k = torch.zeros((2, 8, 64), device="cuda", dtype=torch.float16)
    out = torch.zeros((4, 64), device="cuda")
    c = ctx()
    assert c.attention_gen(q, k, k, out, 3, 8, 8, check=False) == A.ERR_INVALID          # 4 % 3
    assert c.attention_gen(q, k, k, out, 2, 0, 8, check=False) == A.ERR_INVALID          # empty
    assert c.attention_gen(q, k, k, out, 2, 9, 8, check=False) == A.ERR_INVALID          # > capacity
    q96 = torch.zeros((4, 96), device="cuda")
    assert c.attention_gen(q96, k, k, q96.clone(), 2, 8, 8, check=False) == A.ERR_UNSUPPORTED
    sc = torch.zeros((4, 4), device="cuda")
    assert c.attention_gen(q, k, k, out, 2, 8, 8, scores=sc, score_stride=4, check=False) == A.ERR_INVALID
    assert "score_stride" in c.last_error()


@pytest.mark.parametrize("hq,hkv,d,L", [(8, 2, 64, 1023), (8, 2, 64, 1025), (12, 2, 128, 2047), (12, 2, 128, 2500),
                                        (32, 8, 128, 300), (24, 2, 128, 1531), (32, 2, 64, 4097), (16, 2, 128, 66)])
def test_scores_stored_inside_the_token_loop(hq, hkv, d, L):
    # Chunks too long for the LDS stage (beyond ~100K tokens at wide groups) write their logits from
    # inside the token loop; a context created under ARGUS_HIP_SCORES=direct takes that path at test
    # sizes.  Odd strides, rows cut inside a lane's token group, groups wider than eight heads.
    cap = L + 19
    q = normal((hq, d), 42 + L)
    k, v = f16(normal((hkv, cap, d), 137 + L)), f16(normal((hkv, cap, d), 53 + L))
    got, sc = run_decode(q, k, v, hkv, L, cap, scores=True, score_stride=cap, context=direct_ctx())
    assert direct_ctx().last_decode_plan()["staged_scores"] == 0, "logits were staged in LDS after all"
    ref, p = O.attention_gen(q, k, v, hkv, L, cap, scores=True, scores_stride=cap)
    check_attention_out(got, ref, "out")
    check_scores(sc[:, :L], p[:, :L], "scores")
    assert np.all(sc[:, L:] == -7.0), "score columns beyond cache_seq_len must stay untouched"
