"""Pins the oracle's PFA side channel (prefill_attention_scores) with the checks the reference's own
tests make (engine/src/kv/standard_format.rs:3201-3900): an independent float64 eager softmax over the
MHA/GQA x SeqMajor/HeadMajor x windowed/full matrix, the row-sum property, and the per-row relations."""
import numpy as np
import pytest

import oracle as O


def fixture(nq, nkv, layout, head_dim, seq_len, cache_seq_len, kv_capacity):
    # pfa_fixture, standard_format.rs:3513-3537
    q = ((np.arange(seq_len * nq * head_dim) % 13).astype(np.float32) - 6.0) * np.float32(0.1)
    if layout == "seq":
        k_pos_stride, kv_head_stride, k_len = nkv * head_dim, head_dim, cache_seq_len * nkv * head_dim
    else:
        k_pos_stride, kv_head_stride, k_len = head_dim, kv_capacity * head_dim, nkv * kv_capacity * head_dim
    k = ((np.arange(k_len) % 17).astype(np.float32) - 8.0) * np.float32(0.07)
    return q.reshape(seq_len, nq, head_dim), k, k_pos_stride, kv_head_stride


def eager_f64(q, k, nq, nkv, d, seq_len, prefix, kps, khs, q_start, q_window, window):
    """Independent reference: full logit rows and a textbook softmax in float64, returning the per-row
    per-head probabilities [qwin, nq, prefix]."""
    qwin = min(q_window, seq_len)
    out = np.zeros((qwin, nq, prefix))
    g = nq // nkv
    for h in range(nq):
        for step, r in enumerate(range(seq_len - qwin, seq_len)):
            p = q_start + r
            lo = 0 if window is None else max(0, p - max(window - 1, 0))
            keys = np.arange(lo, p + 1)
            rows = np.stack([k[kp * kps + (h // g) * khs: kp * kps + (h // g) * khs + d] for kp in keys]).astype(np.float64)
            logit = rows @ q[r, h].astype(np.float64) / np.sqrt(d)
            e = np.exp(logit - logit.max())
            out[step, h, lo:p + 1] = e / e.sum()
    return out


MATRIX = [(4, 4, "seq"), (4, 2, "seq"), (4, 4, "head"), (4, 2, "head")]


@pytest.mark.parametrize("nq,nkv,layout", MATRIX)
@pytest.mark.parametrize("window", [None, 4])
def test_sum_matches_eager_f64(nq, nkv, layout, window):
    # pfa_matches_eager_softmax_reference (3328-3395): tolerance 1e-4 absolute
    d, seq_len, q_window, cap = 8, 6, 3, 16
    q, k, kps, khs = fixture(nq, nkv, layout, d, seq_len, seq_len, cap)
    got = np.zeros((nq, seq_len), np.float32)
    O.prefill_attention_scores(q, k, nq, nkv, d, seq_len, seq_len, kps, khs, 0, q_window, window, sum_out=got)
    want = eager_f64(q, k, nq, nkv, d, seq_len, seq_len, kps, khs, 0, q_window, window).sum(0)
    assert np.abs(got - want).max() < 1e-4
    # accumulates: a second call doubles the buffer
    O.prefill_attention_scores(q, k, nq, nkv, d, seq_len, seq_len, kps, khs, 0, q_window, window, sum_out=got)
    assert np.abs(got - 2 * want).max() < 2e-4


@pytest.mark.parametrize("q_window", [1, 3])
def test_row_sum_property(q_window):
    # pfa_softmax_sum_property (3463-3509)
    d, seq_len, nq, nkv = 4, 5, 2, 1
    q = (((np.arange(seq_len * nq * d) % 7).astype(np.float32) - 3.0) * np.float32(0.2)).reshape(seq_len, nq, d)
    k = ((np.arange(seq_len * nkv * d) % 5).astype(np.float32) - 2.0) * np.float32(0.3)
    out = np.zeros((nq, seq_len), np.float32)
    O.prefill_attention_scores(q, k, nq, nkv, d, seq_len, seq_len, nkv * d, d, 0, q_window, None, sum_out=out)
    assert np.abs(out.sum(1) - min(q_window, seq_len)).max() < 1e-4


@pytest.mark.parametrize("nq,nkv,layout", MATRIX)
@pytest.mark.parametrize("window", [None, 4])
def test_per_row_relations(nq, nkv, layout, window):
    d, seq_len, q_window, cap = 8, 6, 3, 16
    q, k, kps, khs = fixture(nq, nkv, layout, d, seq_len, seq_len, cap)
    summed = np.zeros((nq, seq_len), np.float32)
    per_head = np.zeros((q_window, nq, seq_len), np.float32)
    O.prefill_attention_scores(q, k, nq, nkv, d, seq_len, seq_len, kps, khs, 0, q_window, window,
                               sum_out=summed, per_row=per_head, per_head=True)
    # pfa_per_row_per_head_sums_to_v1_bit_exact (3539-3603): steps summed in order == sum_out, bit for bit
    acc = np.zeros_like(summed)
    for step in range(q_window):
        acc += per_head[step]
    assert np.array_equal(acc, summed)
    # pfa_per_row_each_step_is_a_distribution (3672-3745)
    assert np.abs(per_head.sum(2) - 1.0).max() < 1e-5
    # causal: nothing beyond the row's own position
    for step, r in enumerate(range(seq_len - q_window, seq_len)):
        assert (per_head[step, :, r + 1:] == 0).all()
    # independent values
    want = eager_f64(q, k, nq, nkv, d, seq_len, seq_len, kps, khs, 0, q_window, window)
    assert np.abs(per_head - want).max() < 1e-5
    # pfa_per_row_head_mean_matches_head_reduced_v1 (3605-3670): head mean == mean over heads of per-head
    mean = np.zeros((q_window, seq_len), np.float32)
    O.prefill_attention_scores(q, k, nq, nkv, d, seq_len, seq_len, kps, khs, 0, q_window, window,
                               per_row=mean, per_head=False)
    assert np.abs(mean - per_head.mean(1)).max() < 1e-6


def test_chunked_prefill_offsets_and_window_clamp():
    # q_start_pos > 0 (second chunk), q_window larger than the chunk, random data
    rng = np.random.default_rng(5)
    nq, nkv, d, seq_len, prefix, q_start = 6, 2, 16, 5, 23, 18
    q = rng.standard_normal((seq_len, nq, d)).astype(np.float32)
    k = rng.standard_normal(prefix * nkv * d).astype(np.float32)
    out = np.zeros((nq, prefix), np.float32)
    O.prefill_attention_scores(q, k, nq, nkv, d, seq_len, prefix, nkv * d, d, q_start, 64, None, sum_out=out)
    want = eager_f64(q, k, nq, nkv, d, seq_len, prefix, nkv * d, d, q_start, 64, None).sum(0)
    assert np.abs(out - want).max() < 1e-5
    assert np.abs(out.sum(1) - seq_len).max() < 1e-4
