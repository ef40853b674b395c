"""GPU parity: argus_hip_attention_gen_desc -- attention over caches of arbitrary descriptor blocks,
in-kernel, against the oracle's composition (decode_via_descriptor, then the scalar F32 attention:
engine/src/kv/standard_format.rs:538-643 with engine/src/format/dtype_layout.rs:102-166)."""
import numpy as np
import pytest

import oracle as O
from gpu_util import check_attention_out, check_scores, ctx, dev, host, normal

pytestmark = pytest.mark.gpu

N, F, FM = O.PACK_NIBBLE, O.SCALE_F16, O.SCALE_F16_MIN
# (block_elems, bits, scale layout, packing): none of them is one of the four named formats
DESCS = [(16, 4, F, N), (64, 4, F, N), (8, 4, FM, N), (16, 3, F, N), (64, 4, FM, N), (16, 8, F, O.PACK_BYTE),
         (64, 8, F, O.PACK_BYTE), (8, 8, F, O.PACK_BYTE), (16, 2, FM, O.PACK_QUAD), (64, 2, FM, O.PACK_QUAD),
         (8, 2, FM, O.PACK_QUAD), (32, 3, FM, N)]


def blocks(desc, n_blocks, seed):
    """random codes under scales (and minima) that decode to N(0,1)-like values"""
    rng = np.random.default_rng(seed)
    bb = O.desc_block_bytes(desc)
    raw = rng.integers(0, 256, size=(n_blocks, bb), dtype=np.uint8)
    levels = 2 ** desc[1] - 1
    d = rng.uniform(2.0, 5.0, n_blocks) / levels
    raw[:, 0:2] = d.astype(np.float16).view(np.uint8).reshape(n_blocks, 2)
    if desc[2] == FM:
        m = -0.5 * levels * d + rng.uniform(-0.2, 0.2, n_blocks)
        raw[:, 2:4] = m.astype(np.float16).view(np.uint8).reshape(n_blocks, 2)
    return raw.reshape(-1)


def run(desc, hq, hkv, d, L, cap, head_major=True, scores=True, softcap=0.0, kv_start=0, index=False, seed=1):
    import argus_hip as A
    be = desc[0]
    kr = blocks(desc, hkv * cap * d // be, seed + 1)
    vr = blocks(desc, hkv * cap * d // be, seed + 2)
    q = normal((hq, d), seed) * np.float32(0.5)
    idx = np.random.default_rng(seed).choice(cap, L, replace=False).astype(np.int32) if index else None
    out = dev(np.full((hq, d), np.nan, np.float32))
    sc = dev(np.full((hq, L + 3), -7.0, np.float32)) if scores else None
    ctx().attention_gen(dev(q), dev(kr), dev(vr), out, hkv, L, cap, layout=A.HEAD_MAJOR if head_major else A.SEQ_MAJOR,
                        scores=sc, score_stride=L + 3 if scores else 0, softcap=softcap, kv_start=kv_start,
                        kv_index=dev(idx) if index else None, desc=desc)
    what = "desc %s Hq%d Hkv%d d%d L%d cap%d %s" % (desc, hq, hkv, d, L, cap, "HM" if head_major else "SM")
    if kv_start:
        bb = O.desc_block_bytes(desc)
        rb = d // be * bb
        kr = kr.reshape(hkv, cap, rb)[:, kv_start:].reshape(-1)
        vr = vr.reshape(hkv, cap, rb)[:, kv_start:].reshape(-1)
        cap -= kv_start
    ref = O.attention_gen_blocks(q, kr, vr, desc, hkv, L, cap, head_major=head_major, scores=scores, softcap=softcap, kv_index=idx)
    if scores:
        check_attention_out(host(out), ref[0], what)
        got = host(sc)
        check_scores(got[:, :L], ref[1], what)
        assert (got[:, L:] == -7.0).all(), what
    else:
        check_attention_out(host(out), ref, what)
    return ctx().last_decode_plan()


@pytest.mark.parametrize("desc", DESCS)
def test_every_block_descriptor_is_attended_in_kernel(desc):
    for hq, hkv, d, L in ((8, 2, 64, 333), (32, 8, 128, 1025), (8, 4, 256, 200), (5, 1, 128, 77)):
        if d % desc[0]:
            continue
        plan = run(desc, hq, hkv, d, L, L + 13, seed=L)
        assert plan["kernel"] == 0  # the vector-ALU kernel, rows decoded in registers


def test_layouts_windows_index_lists_softcap_wide_groups():
    run((16, 4, F, N), 8, 2, 128, 500, 640, head_major=False, seed=3)
    run((16, 4, F, N), 8, 2, 128, 500, 640, kv_start=100, seed=4)
    run((64, 8, F, O.PACK_BYTE), 16, 4, 64, 300, 512, index=True, seed=5)
    run((8, 2, FM, O.PACK_QUAD), 14, 2, 64, 1000, 1024, softcap=5.0, seed=6)
    run((16, 4, FM, N), 24, 2, 128, 200, 256, seed=7)          # 12 query heads per KV head: two head tiles
    run((16, 4, FM, N), 8, 2, 128, 2000, 2048, scores=False, seed=8)
    run((64, 4, F, N), 8, 8, 64, 5, 8, seed=9)                 # one split, written directly


def test_named_formats_take_the_matrix_core_kernel_and_wide_groups_fall_through():
    for desc in (O.DESC_Q4_0, O.DESC_Q4_1, O.DESC_Q8_0, O.DESC_Q2_0):
        plan = run(desc, 32, 8, 128, 1500, 1536, seed=11)
        assert plan["kernel"] == 2
    plan = run(O.DESC_Q4_0, 40, 2, 64, 300, 320, seed=12)      # 20 heads per KV head: beyond the block kernel
    assert plan["kernel"] == 0


def test_descriptors_outside_the_vocabulary_are_declined():
    import torch
    import argus_hip as A
    q = torch.zeros((4, 64), device="cuda")
    out = torch.zeros((4, 64), device="cuda")
    buf = torch.zeros(1 << 16, device="cuda", dtype=torch.uint8)
    for desc in ((1, 16, O.SCALE_NONE, O.PACK_DENSE),   # raw f16: no block form
                 (32, 4, O.SCALE_NONE, N),              # no scale
                 (128, 4, F, N),                        # block beyond 64 elements
                 (12, 4, F, N),                         # not a multiple of 8
                 (32, 5, F, N), (32, 4, F, O.PACK_QUAD), (32, 2, F, O.PACK_QUAD), (32, 4, 7, N), (32, 4, F, 9),
                 (48, 4, F, N)):                        # head_dim 64 is not whole 48-element blocks
        rc = ctx().attention_gen(q, buf, buf, out, 2, 8, 8, desc=desc, check=False)
        assert rc == A.ERR_UNSUPPORTED, desc
        assert "declined" in ctx().last_error()
