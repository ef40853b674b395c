"""Pins of the H2O keep-spec and of the in-place compaction restated in the oracle: the reference's own
known answers (crates/techniques/h2o/src/lib.rs:428-516), a brute-force stable top-k written
independently here, and the gather definition of compaction (engine/src/kv/naive_reference.rs)."""
import numpy as np

import oracle as O


def brute_keep(current, prefix, recent, heavy, score):
    """[0, prefix) + top-`heavy` of the middle by descending score, ties in position order, re-sorted
    ascending + [recent_start, current): written from the doc comment of KeepTopK, not from the oracle."""
    prefix = min(prefix, current)
    recent_start = max(current - recent, prefix) if current >= recent else prefix
    middle = list(range(prefix, recent_start))
    middle.sort(key=lambda p: -float(score[p]))  # Python's sort is stable: ties keep position order
    return list(range(prefix)) + sorted(middle[:heavy]) + list(range(recent_start, current))


def test_reference_known_answers():
    # within_absolute_budget_is_noop: current 10 == 0 + 4 + 6
    assert O.h2o_keep_spec(10, 4, 6) is None
    # score_free_keeps_recency: the last hh + recent = 10 of 20
    kind, keep = O.h2o_keep_spec(20, 4, 6)
    assert kind == "layer" and keep.tolist() == list(range(10, 20))
    # score_based_absolute_heavy_and_recent
    imp = np.zeros(20, np.float32)
    imp[5], imp[9], imp[2] = 10.0, 9.0, 1.0
    kind, keep = O.h2o_keep_spec(20, 2, 4, importance=imp)
    assert kind == "layer" and keep.tolist() == [5, 9, 16, 17, 18, 19]
    # per_head_ranks_independently: hh 3 / recent 3, head 0 prefers 5,6,7 and head 1 prefers 10,11,12
    hs = np.zeros((2, 100), np.float32)
    for i, pos in enumerate((5, 6, 7)):
        hs[0, pos] = 10.0 - i
    for i, pos in enumerate((10, 11, 12)):
        hs[1, pos] = 10.0 - i
    kind, heads = O.h2o_keep_spec(20, 3, 3, head_scores=hs)
    assert kind == "per_head"
    assert heads[0].tolist() == [5, 6, 7, 17, 18, 19] and heads[1].tolist() == [10, 11, 12, 17, 18, 19]


def test_keep_spec_against_brute_force_with_ties_and_short_importance():
    rng = np.random.default_rng(0)
    for case in range(300):
        current = int(rng.integers(1, 90))
        hh, recent, prefix = (int(rng.integers(0, 20)) for _ in range(3))
        # few distinct values: many ties, which the stable sort must break by position
        imp = rng.integers(0, 4, int(rng.integers(0, current + 5))).astype(np.float32)
        got = O.h2o_keep_spec(current, hh, recent, prefix, importance=imp)
        padded = np.zeros(current + 5, np.float32)
        padded[:len(imp)] = imp
        if current <= min(prefix, current) + hh + recent:
            assert got is None, case
            continue
        assert got[0] == "layer" and got[1].tolist() == brute_keep(current, prefix, recent, hh, padded), case
        hs = rng.integers(0, 3, (3, current + 2)).astype(np.float32)
        kind, heads = O.h2o_keep_spec(current, hh, recent, prefix, head_scores=hs)
        assert kind == "per_head" and all(len(h) == len(heads[0]) for h in heads)  # every head keeps the same count
        for h in range(3):
            assert heads[h].tolist() == brute_keep(current, prefix, recent, hh, hs[h]), (case, h)
        kind, keep = O.h2o_keep_spec(current, hh, recent, prefix)
        assert keep.tolist() == brute_keep(current, prefix, hh + recent, 0, padded), case


def test_in_place_compaction_equals_the_gather():
    rng = np.random.default_rng(1)
    for case in range(100):
        hkv, cap, d = int(rng.integers(1, 4)), int(rng.integers(8, 70)), 4
        current = int(rng.integers(1, cap + 1))
        cache = rng.standard_normal((hkv, cap, d)).astype(np.float32)
        keep = np.sort(rng.choice(current, int(rng.integers(1, current + 1)), replace=False))
        want = cache[:, keep]  # the naive gather of engine/src/kv/naive_reference.rs
        got = O.compact_keep_in_place(cache.copy(), keep)
        assert np.array_equal(got[:, :len(keep)], want), case
        assert np.array_equal(O.compact_keep(cache, keep, cap)[:, :len(keep)], want), case
        # per head: only that head moves
        h = int(rng.integers(0, hkv))
        one = O.compact_keep_in_place(cache.copy(), keep, head=h)
        assert np.array_equal(one[h, :len(keep)], want[h])
        for o in range(hkv):
            if o != h:
                assert np.array_equal(one[o], cache[o])
        # runs: consecutive positions merge, runs already in place are skipped
        runs = list(O.keep_batches(keep))
        assert all(s != dst for s, dst, _ in runs)
        assert sum(c for _, _, c in runs) <= len(keep)
    assert list(O.keep_batches([0, 1, 2, 7, 8, 20])) == [(7, 3, 2), (20, 5, 1)]
    assert list(O.keep_batches([0, 1, 2])) == []
