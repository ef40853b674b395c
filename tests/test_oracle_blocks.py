"""The oracle's attention over block-quantised caches (the Q4_0 arm of the scalar CPU backend,
backend/cpu/common.rs:676-850) is pinned here by an independent route: the blocks are unpacked with
a few lines of numpy written from the format definition (quant.rs BlockQ4_0 / BlockQ4_1 / BlockQ8_0:
x = d*(n-8), d*n+m, d*c; element i in the low nibble of byte i, element 16+i in the high nibble;
BlockQ2_0: x = d*n+m, element 4i+k in bits 2k, 2k+1 of byte i) and attended with the float64
textbook softmax attention."""
import numpy as np
import pytest

import oracle as O
import textbook as T
from blocks_util import random_blocks as blocks


def unpack(desc, raw, n_elems):
    bb = O.desc_block_bytes(desc)
    blk = np.asarray(raw, np.uint8).reshape(-1, bb)
    d = blk[:, 0:2].copy().view(np.float16).astype(np.float64)
    if desc == O.DESC_Q8_0:
        x = d * blk[:, 2:].view(np.int8).astype(np.float64)
    elif desc == O.DESC_Q2_0:
        codes = blk[:, 4:]
        n = np.stack([(codes >> (2 * k)) & 3 for k in range(4)], axis=2).reshape(len(blk), 32).astype(np.float64)
        x = d * n + blk[:, 2:4].copy().view(np.float16).astype(np.float64)
    else:
        hdr = 4 if desc == O.DESC_Q4_1 else 2
        codes = blk[:, hdr:]
        n = np.concatenate([codes & 15, codes >> 4], axis=1).astype(np.float64)
        if desc == O.DESC_Q4_1:
            x = d * n + blk[:, 2:4].copy().view(np.float16).astype(np.float64)
        else:
            x = d * (n - 8.0)
    return x.reshape(-1)[:n_elems]


@pytest.mark.parametrize("desc", [O.DESC_Q4_0, O.DESC_Q4_1, O.DESC_Q8_0, O.DESC_Q2_0])
@pytest.mark.parametrize("head_major", [True, False])
def test_against_numpy_unpack_and_textbook_attention(desc, head_major):
    hq, hkv, d, L, cap = 8, 2, 64, 300, 320
    n = hkv * cap * d
    k_raw, v_raw = blocks(desc, n // 32, 1), blocks(desc, n // 32, 2)
    q = np.random.default_rng(3).standard_normal((hq, d)).astype(np.float32)
    out, sc = O.attention_gen_blocks(q, k_raw, v_raw, desc, hkv, L, cap, head_major=head_major, scores=True)
    shape = (hkv, cap, d) if head_major else (cap, hkv, d)
    k = unpack(desc, k_raw, n).reshape(shape)
    v = unpack(desc, v_raw, n).reshape(shape)
    if not head_major:
        k, v = k.transpose(1, 0, 2), v.transpose(1, 0, 2)
    ref_out, ref_p = T.decode_attention(q, k, v, hkv, L)
    assert np.abs(out - ref_out).max() < 1e-5
    assert np.abs(sc - ref_p).max() < 1e-6
    np.testing.assert_allclose(sc.sum(-1), 1.0, rtol=1e-5)


def test_q4_0_unpack_matches_the_descriptor_decode_bit_for_bit():
    raw = blocks(O.DESC_Q4_0, 64, 5)
    got = O.decode_via_descriptor(O.DESC_Q4_0, raw, 64 * 32)
    assert np.array_equal(got, unpack(O.DESC_Q4_0, raw, 64 * 32).astype(np.float32))


def unpack_any(desc, raw, n_elems):
    """Any PerBlockF16[WithMin] x Nibble / Byte / Quad descriptor, written from the doc comments of
    unpack_block_via_descriptor (engine/src/format/dtype_layout.rs:88-101): nibble packing keeps element
    i < n/2 in the low nibble of byte i and element n/2 + i in the high nibble, signed around 2^(bits-1)
    without a minimum, code*scale + min with one; byte packing is i8 * scale; quad packing puts element
    4i + k at bits 2k of byte i."""
    be, bits, scale_layout, packing = desc
    bb = O.desc_block_bytes(desc)
    blk = np.asarray(raw, np.uint8).reshape(-1, bb)
    d = blk[:, 0:2].copy().view(np.float16).astype(np.float64)
    has_min = scale_layout == O.SCALE_F16_MIN
    m = blk[:, 2:4].copy().view(np.float16).astype(np.float64) if has_min else 0.0
    codes = blk[:, 4 if has_min else 2:]
    if packing == O.PACK_BYTE:
        x = d * codes.view(np.int8).astype(np.float64)
    elif packing == O.PACK_QUAD:
        n = np.stack([(codes >> (2 * k)) & 3 for k in range(4)], axis=2).reshape(len(blk), be).astype(np.float64)
        x = d * n + m
    else:
        n = np.concatenate([codes & 15, codes >> 4], axis=1).astype(np.float64)
        x = d * n + m if has_min else d * (n - float(1 << (bits - 1)))
    return x.reshape(-1)[:n_elems]


@pytest.mark.parametrize("desc", [(16, 4, O.SCALE_F16, O.PACK_NIBBLE), (8, 4, O.SCALE_F16_MIN, O.PACK_NIBBLE),
                                  (16, 3, O.SCALE_F16, O.PACK_NIBBLE), (64, 4, O.SCALE_F16_MIN, O.PACK_NIBBLE),
                                  (64, 8, O.SCALE_F16, O.PACK_BYTE), (8, 8, O.SCALE_F16, O.PACK_BYTE),
                                  (16, 2, O.SCALE_F16_MIN, O.PACK_QUAD), (64, 2, O.SCALE_F16_MIN, O.PACK_QUAD),
                                  (32, 3, O.SCALE_F16_MIN, O.PACK_NIBBLE)])
def test_descriptors_beyond_the_named_formats(desc):
    # the decode floor and the attention composed on it, for descriptors no named format uses
    hq, hkv, d, L, cap = 8, 2, 64, 150, 160
    n = hkv * cap * d
    rng = np.random.default_rng(sum(desc))
    bb = O.desc_block_bytes(desc)
    raw = rng.integers(0, 256, size=(n // desc[0], bb), dtype=np.uint8)
    raw[:, 0:2] = rng.uniform(0.05, 0.3, n // desc[0]).astype(np.float16).view(np.uint8).reshape(-1, 2)
    if desc[2] == O.SCALE_F16_MIN:
        raw[:, 2:4] = rng.uniform(-1.5, 0.0, n // desc[0]).astype(np.float16).view(np.uint8).reshape(-1, 2)
    raw = raw.reshape(-1)
    want = unpack_any(desc, raw, n)
    got = O.decode_via_descriptor(desc, raw, n)
    assert np.allclose(got, want, rtol=1e-6, atol=1e-6)
    q = rng.standard_normal((hq, d)).astype(np.float32)
    out, p = O.attention_gen_blocks(q, raw, raw, desc, hkv, L, cap, scores=True)
    kf = want.reshape(hkv, cap, d)
    ref_out, ref_p = T.decode_attention(q, kf, kf, hkv, L)
    assert np.abs(out - ref_out).max() < 1e-5 * (1.0 + np.abs(ref_out).max())  # f32 sums against f64
    assert np.allclose(p, ref_p, rtol=1e-4, atol=1e-9)
