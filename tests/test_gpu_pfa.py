"""GPU parity: PFA side channel (prefill attention scores on the device) against the oracle."""
import numpy as np
import pytest

import oracle as O
from gpu_util import ctx, dev, host
from test_oracle_pfa import MATRIX, fixture

pytestmark = pytest.mark.gpu


def run_dev(q, k, nq, nkv, d, seq_len, prefix, kps, khs, q_start, q_window, window, want_sum, per_row_shape,
            per_head, k_f16=False, sum_init=None):
    import torch
    kd = dev(k.astype(np.float16) if k_f16 else k)
    s = dev(sum_init if sum_init is not None else np.zeros((nq, prefix), np.float32)) if want_sum else None
    pr = torch.zeros(per_row_shape, device="cuda") if per_row_shape else None
    ctx().prefill_attention_scores(dev(q), kd, nq, nkv, d, seq_len, prefix, kps, khs, q_start, q_window, window,
                                   sum_out=s, per_row=pr, per_head=per_head)
    return (host(s) if s is not None else None), (host(pr) if pr is not None else None)


def close(got, ref):
    # required tolerance for score vectors: 1e-4 relative (the reference's own PFA tests use 1e-4 absolute)
    err = np.abs(got.astype(np.float64) - ref.astype(np.float64))
    assert (err <= 1e-4 * np.abs(ref) + 1e-9).all(), err.max()


@pytest.mark.parametrize("nq,nkv,layout", MATRIX)
@pytest.mark.parametrize("window", [None, 4])
def test_reference_matrix(nq, nkv, layout, window):
    d, seq_len, q_window, cap = 8, 6, 3, 16
    q, k, kps, khs = fixture(nq, nkv, layout, d, seq_len, seq_len, cap)
    ref_s = np.zeros((nq, seq_len), np.float32)
    ref_p = np.zeros((q_window, nq, seq_len), np.float32)
    O.prefill_attention_scores(q, k, nq, nkv, d, seq_len, seq_len, kps, khs, 0, q_window, window, sum_out=ref_s,
                               per_row=ref_p, per_head=True)
    got_s, got_p = run_dev(q, k, nq, nkv, d, seq_len, seq_len, kps, khs, 0, q_window, window, True,
                           (q_window, nq, seq_len), True)
    close(got_s, ref_s)
    close(got_p, ref_p)
    # summing the per-head steps in order reproduces sum_out bit for bit, as in the reference
    acc = np.zeros_like(got_s)
    for step in range(q_window):
        acc += got_p[step]
    assert np.array_equal(acc, got_s)
    ref_m = np.zeros((q_window, seq_len), np.float32)
    O.prefill_attention_scores(q, k, nq, nkv, d, seq_len, seq_len, kps, khs, 0, q_window, window, per_row=ref_m)
    _, got_m = run_dev(q, k, nq, nkv, d, seq_len, seq_len, kps, khs, 0, q_window, window, False, (q_window, seq_len), False)
    close(got_m, ref_m)


@pytest.mark.parametrize("k_f16", [False, True])
@pytest.mark.parametrize("nq,nkv,d,seq_len,prefix,q_start,q_window,window",
                         [(32, 8, 128, 64, 1024, 960, 32, None), (8, 4, 256, 40, 300, 260, 64, 128),
                          (14, 2, 64, 128, 128, 0, 16, None), (16, 2, 128, 48, 333, 285, 32, None),
                          (8, 2, 64, 16, 9300, 9284, 8, None)])  # rows longer than the 8192 keys a workgroup holds in registers
def test_model_shapes_head_major(k_f16, nq, nkv, d, seq_len, prefix, q_start, q_window, window):
    # HeadMajor cache [kv_heads, capacity, d], chunked prefill (q_start_pos > 0), accumulation into a
    # non-zero sum buffer, F16 K compared with the oracle fed the f16-rounded K.
    cap = prefix + 13
    rng = np.random.default_rng(prefix + d)
    q = rng.standard_normal((seq_len, nq, d)).astype(np.float32)
    k = rng.standard_normal((nkv, cap, d)).astype(np.float32)
    k_ref = k.astype(np.float16).astype(np.float32) if k_f16 else k
    init = rng.random((nq, prefix)).astype(np.float32)
    ref_s = init.copy()
    qw = min(q_window, seq_len)
    ref_m = np.zeros((qw, prefix), np.float32)
    O.prefill_attention_scores(q, k_ref.reshape(-1), nq, nkv, d, seq_len, prefix, d, cap * d, q_start, q_window, window,
                               sum_out=ref_s, per_row=ref_m)
    got_s, got_m = run_dev(q, k.reshape(-1), nq, nkv, d, seq_len, prefix, d, cap * d, q_start, q_window, window, True,
                           (qw, prefix), False, k_f16=k_f16, sum_init=init)
    close(got_s, ref_s)
    close(got_m, ref_m)
    assert np.abs((got_s - init).sum(1) - qw).max() < 1e-3  # each row adds a distribution


@pytest.mark.parametrize("k_f16", [False, True])
def test_seq_major_per_head_rows_sum_to_sum_out(k_f16):
    # SeqMajor cache [capacity, kv_heads, d] (key stride = kv_heads * d) on the matrix-core logits path,
    # per-head per-row layout: adding a head's rows in order reproduces sum_out bit for bit.
    nq, nkv, d, seq_len, prefix, q_start, q_window = 12, 4, 128, 40, 700, 660, 24
    cap = prefix + 5
    rng = np.random.default_rng(77)
    q = rng.standard_normal((seq_len, nq, d)).astype(np.float32)
    k = rng.standard_normal((cap, nkv, d)).astype(np.float32)
    k_ref = k.astype(np.float16).astype(np.float32) if k_f16 else k
    ref_s = np.zeros((nq, prefix), np.float32)
    ref_r = np.zeros((q_window, nq, prefix), np.float32)
    O.prefill_attention_scores(q, k_ref.reshape(-1), nq, nkv, d, seq_len, prefix, nkv * d, d, q_start, q_window, None,
                               sum_out=ref_s, per_row=ref_r, per_head=True)
    got_s, got_r = run_dev(q, k.reshape(-1), nq, nkv, d, seq_len, prefix, nkv * d, d, q_start, q_window, None, True,
                           (q_window, nq, prefix), True, k_f16=k_f16)
    close(got_s, ref_s)
    close(got_r, ref_r)
    acc = np.zeros((nq, prefix), np.float32)
    for step in range(q_window):
        acc = acc + got_r[step]
    assert (acc.view(np.uint32) == got_s.view(np.uint32)).all()


def test_nothing_armed_and_errors():
    import argus_hip as A
    import torch
    q = torch.zeros((4, 2, 8), device="cuda")
    k = torch.zeros((4 * 2 * 8,), device="cuda")
    assert ctx().prefill_attention_scores(q, k, 2, 2, 8, 4, 4, 16, 8, 0, 2) == 0
    s = torch.zeros((2, 4), device="cuda")
    assert ctx().prefill_attention_scores(q, k, 2, 3, 8, 4, 4, 16, 8, 0, 2, sum_out=s, check=False) == A.ERR_INVALID
    assert ctx().prefill_attention_scores(q, k, 2, 2, 8, 4, 3, 16, 8, 0, 2, sum_out=s, check=False) == A.ERR_INVALID
