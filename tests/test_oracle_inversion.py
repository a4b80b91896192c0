"""Pins the oracle's inversion, run-length/scan and distinct against numpy routines."""
import numpy as np
import pytest


@pytest.mark.parametrize("n", [0, 1, 2, 63, 64, 65, 1000, 50000])
def test_sort_pairs_is_stable_sort(oracle, n):
    rng = np.random.default_rng(n)
    keys = rng.integers(0, 37, n).astype(np.int32)
    vals = rng.integers(0, 1 << 30, n).astype(np.int32)
    ko, vo = oracle.sort_pairs(keys, vals)
    order = np.argsort(keys, kind="stable")
    assert np.array_equal(ko, keys[order]) and np.array_equal(vo, vals[order])


def test_unique_transits_matches_numpy_unique(oracle):
    rng = np.random.default_rng(3)
    invalid = 500
    for n, frac_invalid in [(0, 0), (1, 0), (1, 1), (100, 0.0), (100, 1.0), (5000, 0.3)]:
        keys = rng.integers(0, invalid, n)
        keys[rng.random(n) < frac_invalid] = invalid
        keys = np.sort(keys).astype(np.int32)
        u, c, o, n_valid = oracle.unique_transits(keys, invalid)
        valid = keys[keys != invalid]
        wu, wi, wc = np.unique(valid, return_index=True, return_counts=True)
        assert n_valid == len(valid)
        assert np.array_equal(u, wu) and np.array_equal(c, wc) and np.array_equal(o, wi)
        # the exclusive scan of the counts is the start offset (nextdoor.cu:1749 asserts the same)
        assert np.array_equal(o, np.concatenate([[0], np.cumsum(wc)[:-1]]).astype(np.int32)[:len(o)])


def test_distinct_is_sort_unique_per_segment(oracle):
    rng = np.random.default_rng(5)
    invalid = 30
    d = oracle.app_desc(oracle.KHOP, 2, [5, 4])
    final = rng.integers(0, invalid + 1, (200, 25)).astype(np.int32)
    out, counts = oracle.distinct(d, final, invalid)
    for s in range(200):
        for k, (lo, hi) in enumerate([(0, 5), (5, 25)]):
            seg = final[s, lo:hi]
            want = np.unique(seg[seg != invalid])
            assert counts[s, k] == len(want)
            assert np.array_equal(out[s, lo:lo + len(want)], want)
            assert np.all(out[s, lo + len(want):hi] == invalid)
    # idempotent
    again, counts2 = oracle.distinct(d, out, invalid)
    assert np.array_equal(again, out) and np.array_equal(counts2, counts)
