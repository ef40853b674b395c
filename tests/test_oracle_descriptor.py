"""Pins the oracle's descriptor-driven block codec (format/dtype_layout.rs) with hand-evaluated blocks,
an independent numpy float32 restatement, round-trip bounds, and the q2_0 == KIVI-Q2 codec identity."""
import numpy as np
import pytest

import oracle as O


def f16b(x):
    return np.array([x], np.float32).astype(np.float16).view(np.uint8)


def test_block_bytes():
    # bytes_for_elems_matches_block_struct_size (dtype_layout.rs:408-440): q4_0 18, q4_1 20, q8_0 34, q2_0 12
    assert [O.desc_block_bytes(d) for d in (O.DESC_Q4_0, O.DESC_Q4_1, O.DESC_Q8_0, O.DESC_Q2_0)] == [18, 20, 34, 12]


def test_decode_known_blocks():
    # q4_0: low nibble -> out[i], high nibble -> out[i + 16], value = (nibble - 8) * scale
    qs = np.array([(i & 15) | (((15 - i) & 15) << 4) for i in range(16)], np.uint8)
    blk = np.concatenate([f16b(0.5), qs])
    out = O.decode_via_descriptor(O.DESC_Q4_0, blk, 32)
    assert np.array_equal(out[:16], (np.arange(16) - 8) * 0.5) and np.array_equal(out[16:], (15 - np.arange(16) - 8) * 0.5)
    # q4_1: unsigned nibble * scale + min
    blk = np.concatenate([f16b(0.25), f16b(-1.0), qs])
    out = O.decode_via_descriptor(O.DESC_Q4_1, blk, 32)
    assert np.array_equal(out[:16], np.arange(16) * 0.25 - 1.0) and np.array_equal(out[16:], (15 - np.arange(16)) * 0.25 - 1.0)
    # q8_0: signed bytes
    q8 = np.arange(-16, 16).astype(np.int8).view(np.uint8)
    out = O.decode_via_descriptor(O.DESC_Q8_0, np.concatenate([f16b(0.125), q8]), 32)
    assert np.array_equal(out, np.arange(-16, 16) * 0.125)
    # q2_0: 4 per byte, LSB first, value = q * scale + min
    q2 = np.array([0b11100100] * 8, np.uint8)
    out = O.decode_via_descriptor(O.DESC_Q2_0, np.concatenate([f16b(2.0), f16b(1.0), q2]), 32)
    assert np.array_equal(out, np.tile([1.0, 3.0, 5.0, 7.0], 8))


def np_encode_q4_0(x):
    x = x.astype(np.float32).reshape(-1, 32)
    out = []
    for s in x:
        d = np.float32(np.abs(s).max()) / np.float32(7.0)
        idv = np.float32(0.0) if d == 0 else np.float32(1.0) / d
        t = s * idv
        v = np.clip(np.sign(t) * np.floor(np.abs(t) + np.float32(0.5)), -8, 7).astype(np.int32) + 8
        out.append(np.concatenate([np.array([d], np.float32).astype(np.float16).view(np.uint8),
                                   (v[:16] | (v[16:] << 4)).astype(np.uint8)]))
    return np.concatenate(out)


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_encode_q4_0_matches_numpy_and_round_trips(seed):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal(32 * 40).astype(np.float32)
    x[:32] = 0.0                      # all-zero block: d == 0, id == 0
    x[32:64] = np.round(x[32:64] * 4) / 4  # ties in round()
    x[64] = 50.0                      # outlier
    enc = O.encode_via_descriptor(O.DESC_Q4_0, x)
    assert np.array_equal(enc, np_encode_q4_0(x))
    dec = O.decode_via_descriptor(O.DESC_Q4_0, enc, x.size)
    d = enc.reshape(-1, 18)[:, :2].copy().view(np.float16).astype(np.float32).repeat(32)
    # |x| <= 7 d is reproduced within d/2 (+ the f16 rounding of d); the block maximum itself within d
    assert (np.abs(dec - x) <= 0.5 * d * 1.002 + np.abs(x) * 1e-3 + 1e-7).all()


@pytest.mark.parametrize("seed", [0, 1])
def test_encode_q2_0_is_the_kivi_q2_codec(seed):
    # encode_block_perblockf16withmin_quad mirrors argus_kv_codec::BlockQ2_0::quantize, the block the
    # KIVI Q2 cache stores: both restatements must give the same 12 bytes and the same dequantisation.
    rng = np.random.default_rng(10 + seed)
    x = rng.standard_normal(32 * 25).astype(np.float32)
    x[:32] = 3.0
    enc = O.encode_via_descriptor(O.DESC_Q2_0, x).reshape(-1, 12)
    for i in range(25):
        kb = O.kivi_quantize_block(x[32 * i:32 * i + 32], 2)
        assert np.array_equal(enc[i], kb)
        assert np.array_equal(O.decode_via_descriptor(O.DESC_Q2_0, enc[i], 32), O.kivi_dequantize_block(kb, 2))


def test_encode_outside_writable_floor_is_an_error():
    with pytest.raises(ValueError):
        O.encode_via_descriptor(O.DESC_Q8_0, np.zeros(32, np.float32))
    with pytest.raises(ValueError):
        O.encode_via_descriptor(O.DESC_Q4_1, np.zeros(32, np.float32))
