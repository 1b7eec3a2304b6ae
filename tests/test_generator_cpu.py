"""The numpy Philox4x32-10 used to check the device generator, against the algorithm authors' known-answer vectors."""
import numpy as np

import philox_ref

# Random123 kat_vectors, "philox4x32 10": counter, key -> output
KAT = [
    ((0x00000000, 0x00000000, 0x00000000, 0x00000000), (0x00000000, 0x00000000), (0x6627e8d5, 0xe169c58d, 0xbc57ac4c, 0x9b00dbd8)),
    ((0xffffffff, 0xffffffff, 0xffffffff, 0xffffffff), (0xffffffff, 0xffffffff), (0x408f276d, 0x41c83b0e, 0xa20bc7c6, 0x6d5451fd)),
    ((0x243f6a88, 0x85a308d3, 0x13198a2e, 0x03707344), (0xa4093822, 0x299f31d0), (0xd16cfe09, 0x94fdcceb, 0x5001e420, 0x24126ea1)),
]


def test_philox_known_answers():
    for ctr, key, want in KAT:
        got = philox_ref.philox4x32_10(np.array([ctr], np.uint32), key)[0]
        assert tuple(int(x) for x in got) == want


def test_words_addressing_matches_the_counter_layout():
    # block b of the word stream is the generator at counter (first_block + b, counter_hi), key = seed
    ctr, key, want = KAT[2]
    seed = key[0] | (key[1] << 32)
    first_block = ctr[0] | (ctr[1] << 32)
    counter_hi = ctr[2] | (ctr[3] << 32)
    w = philox_ref.words(8, seed, first_block - 1, counter_hi)
    assert tuple(int(x) for x in w[4:8]) == want
    # the all-ones vector: the block index wraps modulo 2^64
    ctr, key, want = KAT[1]
    w = philox_ref.words(4, 0xffffffffffffffff, 0xffffffffffffffff, 0xffffffffffffffff)
    assert tuple(int(x) for x in w) == want
