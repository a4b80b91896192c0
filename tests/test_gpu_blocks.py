"""GPU parity of the building blocks (Philox fill, inversion sort, run-length/scan)
against the CPU oracle, through the C ABI."""
import numpy as np
import pytest

import nextdoor_amd as nd

pytestmark = pytest.mark.gpu


def test_philox_fill_matches_oracle(oracle):
    seed, step, first = 0x299f31d0a4093822, 7, (1 << 33) + 5
    got = nd.philox_fill_uniform(seed, step, first, 1000, 6)
    for slot in range(0, 1000, 37):
        for d in range(6):
            assert got[slot, d] == oracle.uniform(seed, first + slot, step, d)
    assert got.min() >= 0.0 and got.max() < 1.0


SIZES = [1, 2, 63, 64, 65, 255, 256, 257, 4095, 4096, 4097, 12289, 1000003]


@pytest.mark.parametrize("bits", [1, 8, 9, 16, 23])
def test_sort_pairs_matches_stable_sort(oracle, bits):
    rng = np.random.default_rng(bits)
    for n in SIZES:
        print("sort n", n, "bits", bits, flush=True)
        keys = rng.integers(0, 1 << bits, n).astype(np.int32)
        if n > 10:
            keys[rng.integers(0, n, n // 5)] = (1 << bits) - 1  # a heavy last bucket
        vals = rng.integers(0, 1 << 31, n).astype(np.int32)
        ko, vo = nd.sort_pairs(keys, vals, bits)
        if n <= 70000:
            wk, wv = oracle.sort_pairs(keys, vals)
        else:
            order = np.argsort(keys, kind="stable")
            wk, wv = keys[order], vals[order]
        assert np.array_equal(ko, wk) and np.array_equal(vo, wv)
        # value = index when no values are given
        ko2, vo2 = nd.sort_pairs(keys, None, bits)
        assert np.array_equal(ko2, wk) and np.array_equal(vo2, np.argsort(keys, kind="stable").astype(np.int32))


def test_sort_ignores_bits_above_key_bits():
    keys = np.array([0x105, 0x003, 0x204, 0x001], np.int32)
    ko, vo = nd.sort_pairs(keys, None, 8)
    assert list(ko) == [0x001, 0x003, 0x204, 0x105] and list(vo) == [3, 1, 2, 0]


def test_sort_empty():
    ko, vo = nd.sort_pairs(np.zeros(0, np.int32), None, 8)
    assert len(ko) == 0 and len(vo) == 0


@pytest.mark.parametrize("n,frac_invalid", [(1, 0.0), (1, 1.0), (100, 0.0), (100, 1.0), (2048, 0.2), (2049, 0.0),
                                            (100000, 0.3), (1000003, 0.05)])
def test_unique_transits_matches_oracle(oracle, n, frac_invalid):
    rng = np.random.default_rng(n)
    invalid = 5000
    keys = rng.zipf(1.5, n) % invalid
    keys[rng.random(n) < frac_invalid] = invalid
    keys = np.sort(keys).astype(np.int32)
    u, c, o, n_valid = nd.unique_transits(keys, invalid)
    wu, wc, wo, w_valid = oracle.unique_transits(keys, invalid)
    assert n_valid == w_valid
    assert np.array_equal(u, wu) and np.array_equal(c, wc) and np.array_equal(o, wo)
