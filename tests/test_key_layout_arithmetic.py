"""The sort's first pass finds key i of a segmented input (seg_len keys at the start of every row of
`pitch` words, nd_radix_sort.hpp: KeyLayout) without a division: i / seg_len is the upper 64 bits of
i * magic, magic = floor((2^64 - 1) / seg_len) + 1.  The identity the device code relies on, for
every i below 2^32 (a sort takes at most 2^32 - 1 keys) and every segment length from 2 up."""
import random


def magic_for(seg_len):
    return ((1 << 64) - 1) // seg_len + 1


def test_multiply_high_is_the_quotient_for_every_32_bit_index():
    rng = random.Random(7)
    lengths = [2, 3, 4, 5, 7, 16, 25, 250, 275, 1000, 65535, 65536, (1 << 31) - 1, (1 << 31), (1 << 32) - 1]
    lengths += [rng.randrange(2, 1 << 32) for _ in range(3000)]
    for d in lengths:
        m = magic_for(d)
        assert m < (1 << 64)  # fits the 64-bit field (only a segment length of 1 would not)
        edge = [0, 1, d - 1, d, d + 1, 2 * d - 1, 2 * d, (1 << 32) - 1, (1 << 32) - 2]
        for i in edge + [rng.randrange(0, 1 << 32) for _ in range(100)]:
            if i < (1 << 32):
                assert (i * m) >> 64 == i // d, (i, d)


def test_position_in_the_rows():
    # key i sits at row * pitch + (i - row * seg_len): the k-hop shape (25 ids at the start of 275-id rows)
    seg_len, pitch = 25, 275
    m = magic_for(seg_len)
    for i in (0, 24, 25, 26, 49, 50, 52428799):
        row = (i * m) >> 64
        assert row * pitch + (i - row * seg_len) == (i // seg_len) * pitch + i % seg_len
