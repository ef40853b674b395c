"""Synthetic block-quantised rows for the q4_0 / q4_1 / q8_0 / q2_0 tests: uniformly random codes with
scales (and minima) sized so that the decoded values look like N(0, 1) data of that format."""
import numpy as np

import oracle as O


def random_blocks(desc, n_blocks, seed):
    rng = np.random.default_rng(seed)
    bb = O.desc_block_bytes(desc)
    raw = rng.integers(0, 256, size=(n_blocks, bb), dtype=np.uint8)
    if desc == O.DESC_Q8_0:
        d = rng.uniform(0.005, 0.02, n_blocks)       # codes -128..127
    elif desc == O.DESC_Q2_0:
        d = rng.uniform(0.8, 1.6, n_blocks)          # codes 0..3
    else:
        d = rng.uniform(0.1, 0.3, n_blocks)          # codes -8..7 or 0..15
    raw[:, 0:2] = d.astype(np.float16).view(np.uint8).reshape(n_blocks, 2)
    if desc[2] == O.SCALE_F16_MIN:
        m = -0.5 * (2 ** desc[1] - 1) * d + rng.uniform(-0.2, 0.2, n_blocks)
        raw[:, 2:4] = m.astype(np.float16).view(np.uint8).reshape(n_blocks, 2)
    return raw.reshape(-1)
