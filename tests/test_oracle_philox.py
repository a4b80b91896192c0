"""Pins the oracle's random numbers: Random123 known-answer vectors for Philox4x32-10,
the (slot, step, draw) -> counter/key layout, the [0,1) mapping and rand_int."""
import numpy as np


# Random123 kat_vectors, philox4x32 with 10 rounds: (counter, key, expected)
KAT = [
    ((0, 0, 0, 0), (0, 0), (0x6627e8d5, 0xe169c58d, 0xbc57ac4c, 0x9b00dbd8)),
    ((0xffffffff,) * 4, (0xffffffff,) * 2, (0x408f276d, 0x41c83b0e, 0xa20bc7c6, 0x6d5451fd)),
    ((0x243f6a88, 0x85a308d3, 0x13198a2e, 0x03707344), (0xa4093822, 0x299f31d0),
     (0xd16cfe09, 0x94fdcceb, 0x5001e420, 0x24126ea1)),
]


def test_philox_known_answers(oracle):
    for ctr, key, want in KAT:
        assert tuple(oracle.philox(ctr, key)) == want


def test_uniform_counter_layout(oracle):
    # the pi vector exercises every counter/key word: slot = (c1:c0), step = c2,
    # draw >> 2 = c3, seed = (k1:k0); word index = draw & 3
    ctr, key, want = KAT[2]
    slot = (ctr[1] << 32) | ctr[0]
    seed = (key[1] << 32) | key[0]
    for lane in range(4):
        u = oracle.uniform(seed, slot, ctr[2], ctr[3] * 4 + lane)
        assert u == np.float32((want[lane] >> 8) * 2.0 ** -24)
    # zero vector
    assert oracle.uniform(0, 0, 0, 0) == np.float32((0x6627e8d5 >> 8) * 2.0 ** -24)


def test_uniform_range_and_mean(oracle):
    us = np.array([oracle.uniform(42, s, 3, d) for s in range(2000) for d in range(5)], dtype=np.float64)
    assert us.min() >= 0.0 and us.max() < 1.0
    assert abs(us.mean() - 0.5) < 0.02
    # all representable values are multiples of 2^-24
    assert np.all((us * 2 ** 24) == np.floor(us * 2 ** 24))


def test_rand_int_closed_forms(oracle):
    assert oracle.rand_int(0.0, 10) == 0
    assert oracle.rand_int(0.5, 10) == 5
    assert oracle.rand_int(0.999, 1) == 0
    top = 1.0 - 2.0 ** -24
    # powers of two are exact: floor(k * n / 2^24)
    for n in (1, 2, 64, 4096, 1 << 20, 1 << 24):
        for k in (0, 1, 12345, (1 << 23), (1 << 24) - 1):
            assert oracle.rand_int(k * 2.0 ** -24, n) == (k * n) >> 24
    # general n: the float32 product, truncated, clamped to n - 1
    rng = np.random.default_rng(0)
    for n in [3, 7, 25, 1000, 56944, 4194304, 16777217, (1 << 25) + 6, 2 ** 31 - 1]:
        for u in list(rng.integers(0, 1 << 24, 50) * 2.0 ** -24) + [0.0, top]:
            want = min(int(np.float32(u) * np.float32(n)), n - 1)
            got = oracle.rand_int(u, n)
            assert got == want and 0 <= got <= n - 1
    # curand_uniform can return exactly 1.0; the clamp is what keeps the index in range
    assert oracle.rand_int(1.0, 17) == 16


def test_grouped_stream_is_the_plain_stream_rearranged(oracle):
    """Steps with stepSize > 1 take the first draw of four consecutive output slots from one
    block - counter (slot >> 2, step | 2^31, 0), word slot & 3 - and every later draw from the
    slot's own stream, one position earlier.  Stated on ndo_uniform, which the known-answer
    vectors pin: nothing new is computed, only which word goes where."""
    seed = 0x299f31d0a4093822
    for slot in [0, 1, 2, 3, 4, 5, 7, 250, 251, (1 << 34) + 6, (1 << 34) + 7]:
        for step in (0, 1, 99):
            assert oracle.uniform_grouped(seed, slot, step, 0) == oracle.uniform(seed, slot >> 2, step | (1 << 31), slot & 3)
            for d in range(1, 7):
                assert oracle.uniform_grouped(seed, slot, step, d) == oracle.uniform(seed, slot, step, d - 1)
    # the four slots of a group draw the four words of ONE block, which no slot's own stream uses
    firsts = [oracle.uniform_grouped(seed, 8 + i, 3, 0) for i in range(4)]
    assert len(set(firsts)) == 4
    assert firsts == [oracle.uniform(seed, 2, 3 | (1 << 31), i) for i in range(4)]
    us = np.array([oracle.uniform_grouped(42, s, 1, 0) for s in range(4000)], dtype=np.float64)
    assert us.min() >= 0.0 and us.max() < 1.0 and abs(us.mean() - 0.5) < 0.02
