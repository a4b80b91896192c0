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
    # the buffer of a step that draws several outputs per transit: the grouped form of the stream
    first = (1 << 33) + 6  # not a multiple of four: the first group is cut
    got = nd.philox_fill_uniform(seed, step, first, 1000, 3, step_size=10)
    for slot in list(range(0, 12)) + list(range(12, 1000, 37)):
        for d in range(3):
            assert got[slot, d] == oracle.uniform_grouped(seed, first + slot, step, d)


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


def test_sort_of_more_than_16_mi_pairs_matches_stable_sort():
    """Sorts of at least 2^24 pairs run with larger tiles than the sizes above: a ragged last tile,
    a heavy last bucket, given values and generated ones."""
    n, bits = (16 << 20) + 4097, 23
    rng = np.random.default_rng(5)
    keys = rng.integers(0, 1 << bits, n).astype(np.int32)
    keys[rng.integers(0, n, n // 5)] = (1 << bits) - 1
    vals = rng.integers(0, 1 << 31, n).astype(np.int32)
    order = np.argsort(keys, kind="stable")
    print("sort n", n, "bits", bits, flush=True)
    ko, vo = nd.sort_pairs(keys, vals, bits)
    assert np.array_equal(ko, keys[order]) and np.array_equal(vo, vals[order])
    ko, vo = nd.sort_pairs(keys, None, bits)
    assert np.array_equal(ko, keys[order]) and np.array_equal(vo, order.astype(np.int32))


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


def brute_force_classes(keys, degrees, step_size, thresholds):
    """Which runs the workgroup kernel takes, by the stated rule, and how they are cut."""
    need_work, per_item_outputs, cache_edges = thresholds
    per_item = max(per_item_outputs // step_size, 1)
    transits, starts, counts = np.unique(keys, return_index=True, return_counts=True)
    taken, n_items, single, split, refused = {}, 0, 0, 0, 0
    for t, first, count in zip(transits, starts, counts):
        work = int(count) * step_size
        if work < need_work or degrees[t] == 0:
            continue
        if degrees[t] > cache_edges or degrees[t] > 32 * work:
            refused += int(count)
            continue
        k = -(-int(count) // per_item)
        taken[int(t)] = (int(first), int(count))
        n_items += k
        if k > 1:
            split += int(count)
        else:
            single += int(count)
    return taken, n_items, single, split, refused, per_item


@pytest.mark.parametrize("pairs_per_lane", [1, 16])
@pytest.mark.parametrize("step_size", [1, 2, 10, 25, 3000])
def test_run_classification_covers_every_pair_of_a_taken_transit_once(step_size, pairs_per_lane):
    # the binning of transits into kernel classes (src/nextdoor.cu:1520-1802; the reference asserts
    # the same covering at :1745-1749) against a brute-force partition of the sorted map
    rng = np.random.default_rng(11 + step_size)
    thresholds = nd.load_balancing_thresholds()
    n_vertices = 5000
    degrees = rng.integers(0, 40, n_vertices).astype(np.int32)
    degrees[rng.integers(0, n_vertices, 60)] = rng.integers(5000, 30000, 60)  # adjacencies around and beyond the cache
    degrees[rng.integers(0, n_vertices, 40)] = 0
    # short runs everywhere, some long ones (a few beyond one work item), one at each end of the map
    counts = rng.integers(0, 4, n_vertices)
    long_ones = rng.integers(0, n_vertices, 80)
    counts[long_ones] = rng.integers(20, 700, 80)
    counts[rng.integers(0, n_vertices, 6)] = rng.integers(2500, 9000, 6)
    counts[0], counts[n_vertices - 1] = 300, 2100
    keys = np.repeat(np.arange(n_vertices, dtype=np.int32), counts)
    print("classify n", len(keys), "step size", step_size, "lane", pairs_per_lane, flush=True)
    items, wanted, taken, counters = nd.classify_runs(keys, degrees, step_size, pairs_per_lane)
    want_taken, want_items, single, split, refused, per_item = brute_force_classes(keys, degrees, step_size,
                                                                                   thresholds)
    assert wanted == want_items == len(items)
    assert sorted(np.flatnonzero(taken).tolist()) == sorted(want_taken)
    assert counters.tolist() == [len(keys), single, split, refused, want_items]
    covered = np.zeros(len(keys), np.int32)
    for first, count in items:
        assert 1 <= count <= per_item
        assert len(set(keys[first:first + count].tolist())) == 1  # an item never straddles two transits
        covered[first:first + count] += 1
    for t, (first, count) in want_taken.items():
        assert np.all(covered[first:first + count] == 1)
    assert covered.sum() == sum(c for _, c in want_taken.values())  # nothing else is covered


def test_run_classification_of_a_map_without_long_runs_and_of_an_empty_map():
    degrees = np.full(100, 5, np.int32)
    items, wanted, taken, counters = nd.classify_runs(np.arange(100, dtype=np.int32), degrees, 1)
    assert wanted == 0 and not taken.any() and counters.tolist() == [100, 0, 0, 0, 0]
    items, wanted, taken, counters = nd.classify_runs(np.zeros(0, np.int32), degrees, 1)
    assert wanted == 0 and not taken.any()


def test_gather_rate_measurement_orders_the_memory_levels():
    """The measurement behind the bench's request ceiling: a table that fits L2 serves random
    reads faster than one that does not, and bad sizes are refused."""
    small = nd.measure_gather_rate(1 << 20)
    large = nd.measure_gather_rate(1 << 30)
    print("gather rates", small, large, flush=True)
    assert small > large > 1e9
    with pytest.raises(nd.NextDoorError):
        nd.measure_gather_rate(3 << 20)
