"""GPU parity: descriptor-driven block formats (device floor of --kv-format), bit-exact against the oracle."""
import numpy as np
import pytest

import oracle as O
from gpu_util import check_attention_out, ctx, dev, host

pytestmark = pytest.mark.gpu

DESCS = {"q4_0": O.DESC_Q4_0, "q4_1": O.DESC_Q4_1, "q8_0": O.DESC_Q8_0, "q2_0": O.DESC_Q2_0}


def random_blocks(desc, n_blocks, seed):
    rng = np.random.default_rng(seed)
    bb = O.desc_block_bytes(desc)
    raw = rng.integers(0, 256, (n_blocks, bb), dtype=np.uint8)
    hdr = (rng.standard_normal((n_blocks, 2)) * 0.3).astype(np.float16)
    raw[:, :2] = hdr[:, :1].view(np.uint8)
    if desc[2] == O.SCALE_F16_MIN:
        raw[:, 2:4] = hdr[:, 1:].view(np.uint8)
    return raw.reshape(-1)


@pytest.mark.parametrize("name", list(DESCS))
@pytest.mark.parametrize("n_blocks", [1, 257, 4096])
def test_decode_bit_exact(name, n_blocks):
    import torch
    desc = DESCS[name]
    raw = random_blocks(desc, n_blocks, 7 + n_blocks)
    n = n_blocks * 32
    ref = O.decode_via_descriptor(desc, raw, n)
    d32 = torch.full((n + 8,), 9.0, device="cuda")
    d16 = torch.full((n + 8,), 9.0, device="cuda", dtype=torch.float16)
    src = dev(raw)
    ctx().kv_decode_descriptor(desc, src, d32, n)
    ctx().kv_decode_descriptor(desc, src, d16, n)
    g32, g16 = host(d32), host(d16)
    assert np.array_equal(g32[:n].view(np.uint32), ref.view(np.uint32)) and (g32[n:] == 9.0).all()
    assert np.array_equal(g16[:n].view(np.uint16), ref.astype(np.float16).view(np.uint16)) and (g16[n:] == 9.0).all()


@pytest.mark.parametrize("name", ["q4_0", "q2_0"])
def test_encode_bit_exact_and_round_trip(name):
    import torch
    desc = DESCS[name]
    rng = np.random.default_rng(3)
    x = rng.standard_normal(32 * 1000).astype(np.float32)
    x[:32] = 0.0
    x[32:64] = 2.5
    x[64:96] = np.round(x[64:96] * 4) / 4
    x[100] = 80.0
    ref = O.encode_via_descriptor(desc, x)
    out = torch.full((ref.size + 6,), 0xAB, device="cuda", dtype=torch.uint8)
    ctx().kv_encode_descriptor(desc, dev(x), out, x.size)
    got = host(out)
    assert np.array_equal(got[:ref.size], ref) and (got[ref.size:] == 0xAB).all()
    back = torch.zeros(x.size, device="cuda")
    ctx().kv_decode_descriptor(desc, out, back, x.size)
    assert np.array_equal(host(back), O.decode_via_descriptor(desc, ref, x.size))


def test_errors():
    import argus_hip as A
    import torch
    z = torch.zeros(64, device="cuda")
    b = torch.zeros(128, device="cuda", dtype=torch.uint8)
    assert ctx().kv_encode_descriptor(O.DESC_Q8_0, z, b, 32, check=False) == A.ERR_UNSUPPORTED
    assert ctx().kv_encode_descriptor(O.DESC_Q4_1, z, b, 32, check=False) == A.ERR_UNSUPPORTED
    assert ctx().kv_decode_descriptor((1, 16, O.SCALE_NONE, O.PACK_DENSE), b, z, 32, check=False) == A.ERR_UNSUPPORTED
    assert ctx().kv_decode_descriptor(O.DESC_Q4_0, b, z, 33, check=False) == A.ERR_INVALID
    assert ctx().kv_decode_descriptor(O.DESC_Q4_0, b, z, 0) == 0


def test_q4_0_cache_through_the_floor_matches_oracle_attention():
    # A q4_0 HeadMajor KV cache: encode on the device, decode to F16 on the device, decode attention;
    # equals the oracle's attention over the oracle-decoded cache (the reference floor,
    # standard_format.rs:538-643, with the host round trip removed).
    import torch
    hq, hkv, d, L, cap = 8, 2, 128, 300, 320
    rng = np.random.default_rng(12)
    k = rng.standard_normal((hkv, cap, d)).astype(np.float32)
    v = rng.standard_normal((hkv, cap, d)).astype(np.float32)
    q = rng.standard_normal((hq, d)).astype(np.float32)
    n = k.size
    kq = torch.zeros(n // 32 * 18, device="cuda", dtype=torch.uint8)
    vq = torch.zeros_like(kq)
    ctx().kv_encode_descriptor(O.DESC_Q4_0, dev(k), kq, n)
    ctx().kv_encode_descriptor(O.DESC_Q4_0, dev(v), vq, n)
    k16 = torch.zeros((hkv, cap, d), device="cuda", dtype=torch.float16)
    v16 = torch.zeros_like(k16)
    ctx().kv_decode_descriptor(O.DESC_Q4_0, kq, k16, n)
    ctx().kv_decode_descriptor(O.DESC_Q4_0, vq, v16, n)
    out = torch.zeros((hq, d), device="cuda")
    ctx().attention_gen(dev(q), k16, v16, out, hkv, L, cap)
    kd = O.decode_via_descriptor(O.DESC_Q4_0, O.encode_via_descriptor(O.DESC_Q4_0, k), n).reshape(hkv, cap, d)
    vd = O.decode_via_descriptor(O.DESC_Q4_0, O.encode_via_descriptor(O.DESC_Q4_0, v), n).reshape(hkv, cap, d)
    ref = O.attention_gen(q, kd.astype(np.float16), vd.astype(np.float16), hkv, L, cap)
    check_attention_out(host(out), ref)


@pytest.mark.parametrize("case", range(40))
def test_codec_random_shapes_and_alignments(case):
    # Block sizes other than 32, block counts that do not fill a wave, and buffers that start at odd
    # element offsets (which take the one-thread-per-block kernels) against the oracle, bit for bit.
    import torch
    rng = np.random.default_rng(5000 + case)
    block_elems = int(rng.choice([8, 16, 32, 32, 32, 64]))
    kind = int(rng.integers(0, 4))
    desc = [(block_elems, 4, O.SCALE_F16, O.PACK_NIBBLE), (block_elems, 4, O.SCALE_F16_MIN, O.PACK_NIBBLE),
            (block_elems, 8, O.SCALE_F16, O.PACK_BYTE), (block_elems, 2, O.SCALE_F16_MIN, O.PACK_QUAD)][kind]
    n_blocks = int(rng.choice([1, 2, 3, 63, 64, 65, 255, 1000, 4099]))
    n = n_blocks * block_elems
    bb = O.desc_block_bytes(desc)
    raw = rng.integers(0, 256, size=(n_blocks, bb), dtype=np.uint8)
    raw[:, 0:2] = rng.uniform(0.01, 2.0, n_blocks).astype(np.float16).view(np.uint8).reshape(n_blocks, 2)
    if desc[2] == O.SCALE_F16_MIN:
        raw[:, 2:4] = rng.uniform(-3.0, 3.0, n_blocks).astype(np.float16).view(np.uint8).reshape(n_blocks, 2)
    raw = raw.reshape(-1)
    ref = O.decode_via_descriptor(desc, raw, n)
    off = int(rng.choice([0, 0, 1, 3, 4]))  # elements: an odd offset breaks the 16-byte alignment of the rows
    d32 = torch.full((n + off + 8,), 9.0, device="cuda")
    d16 = torch.full((n + off + 8,), 9.0, device="cuda", dtype=torch.float16)
    src = dev(raw)
    ctx().kv_decode_descriptor(desc, src, d32[off:], n)
    ctx().kv_decode_descriptor(desc, src, d16[off:], n)
    g32, g16 = host(d32), host(d16)
    assert np.array_equal(g32[off:off + n].view(np.uint32), ref.view(np.uint32))
    assert (g32[:off] == 9.0).all() and (g32[off + n:] == 9.0).all()
    assert np.array_equal(g16[off:off + n].view(np.uint16), ref.astype(np.float16).view(np.uint16))
    assert (g16[:off] == 9.0).all() and (g16[off + n:] == 9.0).all()
    if kind in (0, 3):  # the two writable formats
        x = (rng.standard_normal(n) * rng.choice([0.01, 1.0, 30.0])).astype(np.float32)
        x[: block_elems] = 0.0
        want = O.encode_via_descriptor(desc, x)
        xs = torch.zeros(n + off, device="cuda")
        xs[off:] = dev(x)
        out = torch.full((want.size + 6,), 0xAB, device="cuda", dtype=torch.uint8)
        ctx().kv_encode_descriptor(desc, xs[off:], out, n)
        got = host(out)
        assert np.array_equal(got[:want.size], want) and (got[want.size:] == 0xAB).all()
