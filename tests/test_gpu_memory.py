"""GPU tests of the memory entry points behind Backend::{write_buffer_range, buffer_shift, copy_slice}
(engine/src/backend.rs:736, 1085-1112, 1119), through the C ABI."""
import numpy as np
import pytest

from gpu_util import ctx, dev, host

pytestmark = pytest.mark.gpu


def shifted(a, src, dst, count):
    """memmove on the host: numpy copies through a temporary when the slices overlap."""
    b = a.copy()
    b[dst:dst + count] = a[src:src + count]
    return b


@pytest.mark.parametrize("dtype", [np.float32, np.float16, np.uint8])
@pytest.mark.parametrize("n,src,dst,count", [
    (4096, 1024, 0, 3072),        # towards the front, overlapping (prefix prune)
    (4096, 0, 1024, 3072),        # towards the back, overlapping
    (4096, 1, 0, 4095),           # by one element
    (4096, 0, 1, 4095),
    (4096, 2048, 0, 2048),        # touching, disjoint
    (5000, 4000, 10, 1000),       # disjoint
    (3_000_001, 7, 0, 2_999_990),  # large move by a few bytes: staged through the workspace
    (3_000_001, 0, 13, 2_999_900),
    (40_000_000, 1_500_000, 0, 38_000_000),  # distance above 1 MiB: direct pieces
    (40_000_000, 0, 1_500_000, 38_000_000),
])
def test_buffer_shift_is_memmove(dtype, n, src, dst, count):
    rng = np.random.default_rng(n + src + dst)
    a = rng.integers(0, 255, n).astype(dtype)
    t = dev(a)
    ctx().buffer_shift(t, src, dst, count)
    assert np.array_equal(host(t), shifted(a, src, dst, count))


def test_residual_ring_shift_after_a_partial_flush():
    # engine/src/kv/quant_window_cache.rs:1820-1841: per KV head, the rows that remain after a flush
    # move to the front of the head's window [kv_heads, res_cap, head_dim] F32; with 96 of 128 rows
    # remaining after a 32-row flush the ranges overlap.
    hkv, res_cap, d, flush, res_pos = 8, 128, 128, 32, 128
    a = np.random.default_rng(0).standard_normal((hkv, res_cap, d)).astype(np.float32)
    t = dev(a)
    remaining = res_pos - flush
    for h in range(hkv):
        base = h * res_cap * d
        ctx().buffer_shift(t, base + flush * d, base, remaining * d)
    want = a.copy()
    want[:, :remaining] = a[:, flush:res_pos]
    assert np.array_equal(host(t), want)


def test_copy_slice_hands_overlapping_ranges_to_the_shift():
    a = np.arange(100000, dtype=np.float32)
    t = dev(a)
    es = 4
    ctx().copy_slice(t.data_ptr(), t.data_ptr() + 100 * es, 90000 * es)
    assert np.array_equal(host(t), shifted(a, 100, 0, 90000))
    u = dev(np.zeros(1000, np.float32))
    ctx().copy_slice(u.data_ptr() + 16, t.data_ptr(), 400)
    assert np.array_equal(host(u)[4:104], host(t)[:100])


def test_write_buffer_range():
    a = np.zeros(1000, np.float32)
    t = dev(a)
    src = np.arange(10, dtype=np.float32)
    ctx().write_buffer_range(t, 40 * 4, src)
    a[40:50] = src
    assert np.array_equal(host(t), a)


def test_workspace_hint_covers_the_announced_call_without_growth():
    # a context created with the session's limits serves its largest call from the workspace it
    # allocated at creation; the plan of that call stays within it
    import torch
    import argus_hip as A
    c = A.Context(0, max_batch=4, max_heads_q=32, max_head_dim=128, max_seq_len=8192)
    b, hq, hkv, d, L = 4, 32, 8, 128, 8192
    g = torch.Generator(device="cuda").manual_seed(1)
    k = torch.randn((b, hkv, L, d), generator=g, device="cuda").half()
    v = torch.randn((b, hkv, L, d), generator=g, device="cuda").half()
    q = torch.randn((b, hq, d), generator=g, device="cuda")
    out = torch.empty_like(q)
    free0 = torch.cuda.mem_get_info()[0]
    c.attention_gen(q, k, v, out, hkv, L, L, batch=b, kv_batch_stride=hkv * L * d)
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free0, "the call allocated device memory"
    out2 = torch.empty_like(q)
    ctx().attention_gen(q, k, v, out2, hkv, L, L, batch=b, kv_batch_stride=hkv * L * d)
    assert torch.equal(out, out2)
    c.close()
