"""GPU parity: argus_hip_flash_attention_prefill (through the C ABI) against the CPU oracle."""
import numpy as np
import pytest

import oracle as O
import textbook as T
from gpu_util import check_attention_out, ctx, dev, host, normal

pytestmark = pytest.mark.gpu


def f16(x):
    return O.f32_to_f16_bits(x).view(np.float16)


def run_prefill(q, k, v, hkv, cache_len, cap, out_dtype=None, window=0, head_major=True, check=True):
    """q [B, S, Hq, d]; k, v [B, Hkv, cap, d].  Returns (rc, out)."""
    import torch
    b, s, hq, d = q.shape
    qd, kd, vd = dev(q), dev(k), dev(v)
    odt = {np.float32: torch.float32, np.float16: torch.float16}[out_dtype or q.dtype.type]
    out = torch.full((b, s, hq, d), float("nan"), dtype=odt, device="cuda")
    rc = ctx().flash_attention_prefill(qd, kd, vd, out, hq, hkv, s, cache_len, d, cap, batch_size=b,
                                       is_head_major=head_major, window=window, check=check)
    return rc, host(out).astype(np.float32)


# engine/tests/test_prefill_flash_attention.rs:240-559 matrix (q_len, Hq, Hkv, d, q_start_pos, window,
# seed) on the tests' LCG data; reference bound NMSE < 1e-4.
CASES = [
    (32, 4, 2, 64, 0, 0, 0x10), (64, 4, 2, 64, 0, 0, 0x11), (127, 4, 2, 64, 0, 0, 0x12),
    (128, 4, 2, 64, 0, 0, 0x20), (129, 4, 2, 64, 0, 0, 0x21), (256, 8, 2, 64, 0, 0, 0x22),
    (512, 32, 8, 64, 0, 0, 0x23), (1024, 12, 2, 128, 0, 0, 0x24), (193, 4, 2, 64, 0, 0, 0x31),
    (205, 4, 2, 64, 0, 0, 0x32), (200, 12, 2, 128, 0, 0, 0x33), (256, 4, 4, 64, 0, 0, 0x40),
    (256, 12, 2, 128, 0, 0, 0x43), (256, 32, 4, 64, 0, 0, 0x44), (512, 4, 2, 64, 0, 64, 0x50),
    (256, 4, 2, 64, 0, 1024, 0x51), (256, 4, 2, 64, 16, 0, 0x60), (100, 8, 4, 256, 0, 0, 0x70),
    (300, 6, 2, 256, 37, 0, 0x71), (333, 14, 2, 64, 5, 100, 0x72), (1, 4, 2, 128, 0, 0, 0x73),
    (1, 4, 2, 64, 200, 0, 0x74),
]


@pytest.mark.parametrize("q_len,hq,hkv,d,qsp,window,seed", CASES)
@pytest.mark.parametrize("kv", ["f16", "f32"])
def test_prefill_reference_matrix(q_len, hq, hkv, d, qsp, window, seed, kv):
    kv_len = qsp + q_len
    cap = kv_len + 3
    q = O.gen_data(q_len * hq * d, seed + 1).reshape(1, q_len, hq, d)
    k = O.gen_data(hkv * cap * d, seed + 2).reshape(1, hkv, cap, d)
    v = O.gen_data(hkv * cap * d, seed + 3).reshape(1, hkv, cap, d)
    if kv == "f16":
        k, v = f16(k), f16(v)
    rc, got = run_prefill(q, k, v, hkv, kv_len, cap, window=window)
    assert rc == 1
    ref = O.prefill_attention(q, k, v, hkv, kv_len, cap, window=window)
    assert T.nmse(got, ref) < 1e-4
    check_attention_out(got, ref)
    r64 = T.prefill_attention(q[0], k[0], v[0], hkv, kv_len, qsp, window)
    check_attention_out(got[0], r64, "vs f64")


def test_prefill_closed_forms():
    # engine/src/kv/standard_format.rs:3095-3199: K = 0, V[p] = p  =>  out[r] = r/2.
    s, hq, hkv, d = 200, 4, 2, 64
    q = normal((1, s, hq, d), 1)
    k = np.zeros((1, hkv, s, d), np.float16)
    v = np.broadcast_to(np.arange(s, dtype=np.float16)[None, None, :, None], (1, hkv, s, d)).copy()
    rc, got = run_prefill(q, k, v, hkv, s, s)
    assert rc == 1
    assert np.abs(got - (np.arange(s) / 2.0)[None, :, None, None]).max() < 1e-3
    # strict causality (engine/tests/test_prefill_flash_attention.rs:234-312): poisoning every key /
    # value above the diagonal must not change any output
    k2 = f16(normal((1, hkv, s, d), 2))
    v2 = f16(normal((1, hkv, s, d), 3))
    _, base = run_prefill(q[:, :100], k2, v2, hkv, 100, s)
    k3, v3 = k2.copy(), v2.copy()
    k3[:, :, 100:], v3[:, :, 100:] = 77.0, -55.0
    _, pois = run_prefill(q[:, :100], k3, v3, hkv, 100, s)
    assert np.array_equal(base, pois)
    # window 1: every row sees only its own key => out == V row
    _, w1 = run_prefill(q, k2, v2, hkv, s, s, window=1)
    want = np.repeat(v2[0].astype(np.float32).transpose(1, 0, 2), hq // hkv, axis=1)
    assert np.abs(w1[0] - want).max() < 1e-6


def test_config2_llama1b_shape_all_f16():
    # benchmark configuration 2: Hq32 Hkv8 d64 S2048 batch 1, f16 Q/K/V N(0,1) seeded, f32 accumulate, f16 out.
    s, hq, hkv, d = 2048, 32, 8, 64
    q = f16(normal((1, s, hq, d), 42))
    k = f16(normal((1, hkv, s, d), 137))
    v = f16(normal((1, hkv, s, d), 53))
    rc, got = run_prefill(q, k, v, hkv, s, s)
    assert rc == 1
    ref = O.prefill_attention(q.astype(np.float32), k, v, hkv, s, s)
    check_attention_out(got, ref)
    # reference-shaped variant: F32 Q / F32 out
    rc, got32 = run_prefill(q.astype(np.float32), k, v, hkv, s, s)
    check_attention_out(got32, ref)


@pytest.mark.parametrize("d", [64, 128])
def test_grid_that_fills_the_device_with_four_wave_workgroups(d):
    # Two sequences of the config-2 shape give 512 workgroups: the launcher then runs one KV group
    # per workgroup (two independent workgroups per compute unit) instead of two groups in one.
    b, s, hq, hkv = 2, 2048, 32, 8
    q = f16(normal((b, s, hq, d), 7))
    k = f16(normal((b, hkv, s, d), 8))
    v = f16(normal((b, hkv, s, d), 9))
    rc, got = run_prefill(q, k, v, hkv, s, s)
    assert rc == 1
    check_attention_out(got, O.prefill_attention(q.astype(np.float32), k, v, hkv, s, s))


@pytest.mark.parametrize("hq,hkv,d,s,b", [(32, 32, 64, 512, 16), (32, 8, 64, 512, 32), (16, 16, 128, 384, 32)])
def test_grid_of_four_workgroups_per_cu_takes_one_query_tile_each(hq, hkv, d, s, b):
    # From 1024 workgroups on (256 CUs) the launcher stops pairing query tiles (n-1-j, j) and gives
    # every workgroup one tile, longest first: many short sequences, ragged last tiles included.
    q = f16(normal((b, s - 5, hq, d), 17))
    k = f16(normal((b, hkv, s, d), 18))
    v = f16(normal((b, hkv, s, d), 19))
    rc, got = run_prefill(q, k, v, hkv, s - 5, s)
    assert rc == 1
    check_attention_out(got, O.prefill_attention(q.astype(np.float32), k, v, hkv, s - 5, s))


def test_batched_prefill_with_capacity_and_offset():
    b, s, hq, hkv, d, cap, csl = 3, 150, 8, 2, 128, 400, 333
    q = normal((b, s, hq, d), 1)
    k = f16(normal((b, hkv, cap, d), 2))
    v = f16(normal((b, hkv, cap, d), 3))
    rc, got = run_prefill(q, k, v, hkv, csl, cap)
    assert rc == 1
    check_attention_out(got, O.prefill_attention(q, k, v, hkv, csl, cap))
    for i in range(b):
        check_attention_out(got[i], T.prefill_attention(q[i], k[i], v[i], hkv, csl, csl - s), "seq %d" % i)


def test_declined_and_invalid_cases():
    import argus_hip as A
    q = normal((1, 8, 4, 64), 1)
    k = f16(normal((1, 2, 8, 64), 2))
    # SeqMajor and unsupported head_dim are declined (Ok(false)): engine/src/backend/cuda_pc.rs:851-860
    rc, _ = run_prefill(q, k, k, 2, 8, 8, head_major=False)
    assert rc == 0
    q96 = normal((1, 8, 4, 96), 1)
    k96 = f16(normal((1, 2, 8, 96), 2))
    rc, _ = run_prefill(q96, k96, k96, 2, 8, 8)
    assert rc == 0
    rc, _ = run_prefill(q, k, k, 3, 8, 8, check=False)
    assert rc == A.ERR_INVALID
    rc, _ = run_prefill(q, k, k, 2, 4, 8, check=False)   # cache_seq_len < seq_len
    assert rc == A.ERR_INVALID
