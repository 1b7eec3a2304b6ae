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


# ---------------------------------------------------------------------------- the configurations' generator (mt19937 + Box-Muller)
def test_synth_engine_is_mt19937():
    """The C++ standard fixes std::mt19937: the 10000th output of a default-seeded (5489) engine is 4123659995; numpy's
    legacy RandomState is the same engine with the same integer seeding."""
    from eddl_amd.synth import Synth
    assert int(Synth(5489).words(10000)[-1]) == 4123659995
    for seed in (0, 1, 42, 2 ** 32 - 1):
        want = np.random.RandomState(seed).randint(0, 2 ** 32, 2000, dtype=np.uint64).astype(np.uint32)
        assert np.array_equal(Synth(seed).words(2000), want)


def test_synth_uniform_and_normal_follow_their_definition():
    from eddl_amd.synth import Synth
    n = 100001
    w = Synth(9).words(n)
    u = (w >> np.uint32(8)).astype(np.float64) * 2.0 ** -24
    assert np.array_equal(Synth(9).uniform((n,), -2.0, 3.0), (-2.0 + 5.0 * u).astype(np.float32))
    w = Synth(9).words(n + 1).reshape(-1, 2)
    u1 = ((w[:, 0] >> np.uint32(8)).astype(np.float64) + 1.0) * 2.0 ** -24
    u2 = (w[:, 1] >> np.uint32(8)).astype(np.float64) * 2.0 ** -24
    r = np.sqrt(-2.0 * np.log(u1))
    z = np.stack([r * np.cos(2 * np.pi * u2), r * np.sin(2 * np.pi * u2)], axis=1).reshape(-1)[:n]
    got = Synth(9).normal((n,), 0.5, 2.0)
    # numpy's log / cos / sin may differ from libm's in the last place of the double, which can move the float by one ulp
    assert np.abs(got - (0.5 + 2.0 * z)).max() <= 4e-7 * (1 + np.abs(z).max() * 2)
    g = got.astype(np.float64)
    assert abs(g.mean() - 0.5) < 5 * 2.0 / np.sqrt(n) and abs(g.std() / 2.0 - 1.0) < 5 / np.sqrt(2 * n)
    # a stream continues across calls; a fill of an odd count starts the next one on a fresh pair
    s = Synth(9)
    a, b = s.normal((3,)), s.normal((2,))
    w = Synth(9).words(6)
    s2 = Synth(9)
    full = s2.normal((4,))
    assert np.array_equal(a, full[:3])
    s3 = Synth(9)
    s3.words(4)
    assert np.array_equal(b, s3.normal((2,)))


def test_model_parameters_are_a_function_of_the_seed_alone():
    from eddl_amd import models
    a = models.init_he_normal(models.conv_bn_relu_pool_block(batch=2, channels=5, size=12, filters=7), 2)
    b = models.init_he_normal(models.conv_bn_relu_pool_block(batch=9, channels=5, size=12, filters=7), 2)
    for la, lb in zip(a.layers, b.layers):
        for k in la.params:
            assert np.array_equal(la.params[k], lb.params[k])
    K = [l for l in a.layers if l.kind == "conv2d"][0].params["K"]
    assert abs(K.std() / np.sqrt(2.0 / 45) - 1.0) < 0.2
    x9 = models.synthetic_input((9, 5, 12, 12), 1002, "normal")
    x2 = models.synthetic_input((2, 5, 12, 12), 1002, "normal")
    assert np.array_equal(x9[:2], x2)   # a smaller batch is the prefix of a larger one
