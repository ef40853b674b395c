"""GPU test of the entry point that allocates nothing: argus_hip_attention_gen_noalloc keeps its
split-KV partials in the library's static device array.  Checked against argus_hip_attention_gen
(same kernels, same split plan: identical results) on two calls in a row, the second smaller, then
over the shapes that take the other kernels, and for the refusal of a call that does not fit."""
import numpy as np
import pytest

import oracle as O
from gpu_util import check_attention_out, check_scores, ctx, dev, host, normal

pytestmark = pytest.mark.gpu


def f16(x):
    return O.f32_to_f16_bits(x).view(np.float16)


def both(q, k, v, hkv, L, cap, scores=False, **kw):
    """(existing entry point, no-alloc entry point) outputs [and scores] for the same inputs."""
    import torch
    res = []
    qd, kd, vd = dev(q), dev(k), dev(v)
    for noalloc in (False, True):
        out = torch.full(q.shape, float("nan"), dtype=torch.float32, device="cuda")
        sc = torch.full(q.shape[:-1] + (cap,), -7.0, dtype=torch.float32, device="cuda") if scores else None
        free0 = torch.cuda.mem_get_info()[0]
        ctx().attention_gen(qd, kd, vd, out, hkv, L, cap, scores=sc, score_stride=cap if scores else 0, noalloc=noalloc, **kw)
        torch.cuda.synchronize()
        if noalloc:
            assert torch.cuda.mem_get_info()[0] == free0, "the no-alloc entry point changed the free device memory"
        res.append((host(out), host(sc) if scores else None))
    return res


def test_two_calls_in_a_row_the_second_smaller():
    hq, hkv, d = 32, 8, 128
    for L, b in ((8192, 4), (1000, 1)):  # the second call leaves most of the first call's partials in the array
        q = normal((b, hq, d), 42 + L)
        k = f16(normal((b, hkv, L, d), 137 + L))
        v = f16(normal((b, hkv, L, d), 53 + L))
        (ref, ref_sc), (got, got_sc) = both(q, k, v, hkv, L, L, scores=True, batch=b, kv_batch_stride=hkv * L * d)
        assert ctx().last_decode_plan()["nsplit"] > 1
        assert np.array_equal(got, ref), "L %d" % L
        assert np.array_equal(got_sc, ref_sc), "L %d scores" % L
        for i in range(b):
            o, p = O.attention_gen(q[i], k[i], v[i], hkv, L, L, scores=True)
            check_attention_out(got[i], o, "L %d seq %d vs oracle" % (L, i))
            check_scores(got_sc[i][:, :L], p, "L %d seq %d vs oracle" % (L, i))


@pytest.mark.parametrize("kind,hq,hkv,d,L", [("f32", 8, 2, 64, 3000), ("f16", 8, 4, 256, 2048), ("f16", 14, 2, 64, 40),
                                             ("q4_0", 32, 8, 128, 4096), ("q8_0", 14, 2, 64, 1500)])
def test_other_kernels_share_the_array(kind, hq, hkv, d, L):
    import argus_hip as A
    q = normal((hq, d), L)
    kw = {}
    if kind in ("q4_0", "q8_0"):
        from blocks_util import random_blocks
        desc = {"q4_0": O.DESC_Q4_0, "q8_0": O.DESC_Q8_0}[kind]
        k = random_blocks(desc, hkv * L * d // 32, L + 1)
        v = random_blocks(desc, hkv * L * d // 32, L + 2)
        kw["kv_dtype"] = getattr(A, kind.upper())
    else:
        k, v = normal((hkv, L, d), L + 1), normal((hkv, L, d), L + 2)
        if kind == "f16":
            k, v = f16(k), f16(v)
    (ref, _), (got, _) = both(q, k, v, hkv, L, L, **kw)
    assert np.array_equal(got, ref)
    (ref, ref_sc), (got, got_sc) = both(q, k, v, hkv, L, L, scores=True, **kw)
    assert np.array_equal(got, ref) and np.array_equal(got_sc, ref_sc)


def test_a_call_beyond_the_array_is_refused_and_the_next_one_works():
    # 4 sequences x 64 heads x 67 splits x (256 + 2) floats = 17.7 MB of partials > 16 MiB
    import torch
    import argus_hip as A
    b, hq, hkv, d, L = 4, 64, 8, 256, 131072
    k = torch.zeros((b, hkv, L, d), device="cuda", dtype=torch.float16)
    q = torch.zeros((b, hq, d), device="cuda")
    out = torch.zeros((b, hq, d), device="cuda")
    sc = torch.zeros((b, hq, L), device="cuda")
    rc = ctx().attention_gen(q, k, k, out, hkv, L, L, scores=sc, score_stride=L, batch=b, kv_batch_stride=hkv * L * d,
                             noalloc=True, check=False)
    assert rc == A.ERR_NOMEM, rc
    assert "static scratch" in ctx().last_error()
    del k, sc
    hq, hkv, d, L = 32, 8, 128, 2048
    q = normal((hq, d), 1)
    kk, vv = f16(normal((hkv, L, d), 2)), f16(normal((hkv, L, d), 3))
    (ref, _), (got, _) = both(q, kk, vv, hkv, L, L)
    assert np.array_equal(got, ref)
