"""Random fills and scalar operations that EDDL's initialisers run on the device (eddlhip_rand_*, eddlhip_mult_scalar,
eddlhip_add_scalar), through the C ABI.

What is pinned and how: the generator is Philox4x32-10, checked word for word against a numpy restatement that
reproduces the algorithm authors' known-answer vectors (test_generator_cpu.py); uniform, signed-uniform and binary
fills are exact float functions of those words and are compared bit for bit; the normal fill is compared with a
float64 Box-Muller of the same words to 2e-6 (device logf / sincosf) and through its moments.  Parity with the
reference's own random STREAMS (cuRAND MRG32k3a on its GPU path, std::mt19937 seeded from std::random_device on its
CPU path) is unpinned by construction: only the distributions are checked, with the bounds stated below.
"""
import ctypes

import numpy as np
import pytest

import philox_ref

pytestmark = pytest.mark.gpu


def test_raw_words_are_philox4x32_10(hip):
    # the authors' known-answer vectors, reached through the entry point's (seed, first_block, counter_hi) addressing
    assert [int(x) for x in hip.rand_words(4, 0, 0, 0)] == [0x6627e8d5, 0xe169c58d, 0xbc57ac4c, 0x9b00dbd8]
    assert [int(x) for x in hip.rand_words(4, 2 ** 64 - 1, 2 ** 64 - 1, 2 ** 64 - 1)] == [0x408f276d, 0x41c83b0e, 0xa20bc7c6, 0x6d5451fd]
    got = hip.rand_words(8, 0x299f31d0a4093822, 0x85a308d3243f6a88 - 1, 0x0370734413198a2e)
    assert [int(x) for x in got[4:]] == [0xd16cfe09, 0x94fdcceb, 0x5001e420, 0x24126ea1]
    rng = np.random.default_rng(11)
    for n in (1, 2, 3, 5, 1023, 65537, 1 << 20):
        seed, first, hi = (int(x) for x in rng.integers(0, 2 ** 63, 3))
        assert np.array_equal(hip.rand_words(n, seed, first, hi), philox_ref.words(n, seed, first, hi)), n


@pytest.mark.parametrize("n", [1, 3, 4, 7, 4096, 100003])
def test_uniform_fills_bit_exact(hip, n):
    seed = 1234 + n
    t = hip.full((n,), np.nan)
    hip.rand_uniform(t, 0.75, seed)
    got = t.numpy()
    assert np.array_equal(got, philox_ref.uniform(n, 0.75, seed))
    assert got.min() >= 0.0 and got.max() < 0.75
    hip.rand_signed_uniform(t, 0.1, seed)
    got = t.numpy()
    assert np.array_equal(got, philox_ref.signed_uniform(n, 0.1, seed))
    assert np.abs(got).max() <= np.float32(0.1)
    hip.rand_binary(t, 0.3, seed)
    assert np.array_equal(t.numpy(), philox_ref.binary(n, 0.3, seed))


def test_fills_are_reproducible_and_seeds_independent(hip):
    n = 1 << 18
    a, b, c = hip.empty((n,)), hip.empty((n,)), hip.empty((n,))
    hip.rand_normal(a, 0.0, 1.0, 7)
    hip.rand_normal(b, 0.0, 1.0, 7)
    hip.rand_normal(c, 0.0, 1.0, 8)
    x, y, z = a.numpy(), b.numpy(), c.numpy()
    assert np.array_equal(x, y)
    assert abs(float(np.corrcoef(x, z)[0, 1])) < 5.0 / np.sqrt(n)
    # a fill into memory that is not 16-byte aligned (one float into a tensor) gives the same values
    big = hip.full((n + 1,), 5.0)
    hip._check(hip.lib.eddlhip_rand_normal(hip.dev, big.ptr + 4, n, 0.0, 1.0, 7))
    out = big.numpy()
    assert out[0] == 5.0 and np.array_equal(out[1:], x)


def test_normal_fill_values_and_moments(hip):
    n = 1 << 22
    t = hip.empty((n,))
    hip.rand_normal(t, 0.5, 2.0, 99)
    got = t.numpy().astype(np.float64)
    want = philox_ref.normal(n, 0.5, 2.0, 99)
    assert np.abs(got - want).max() <= 2e-6 * (1.0 + np.abs(want).max())
    z = (got - 0.5) / 2.0
    se = 1.0 / np.sqrt(n)
    assert abs(z.mean()) < 5 * se                          # mean of n standard normals: sd 1/sqrt(n)
    assert abs(z.var() - 1.0) < 5 * np.sqrt(2.0) * se      # variance: sd sqrt(2/n)
    assert abs((z ** 3).mean()) < 5 * np.sqrt(15.0) * se   # third moment: sd sqrt(15/n)
    assert abs((z ** 4).mean() - 3.0) < 5 * np.sqrt(96.0) * se  # fourth moment: sd sqrt(96/n)
    # tails: P(|z| > 3) = 0.0026998; binomial sd sqrt(p(1-p)/n)
    p = 0.002699796
    assert abs((np.abs(z) > 3).mean() - p) < 5 * np.sqrt(p * (1 - p) / n)
    assert np.isfinite(got).all() and np.abs(z).max() < 6.0  # sqrt(-2 ln 2^-24) = 5.77 is the largest radius


def test_uniform_moments(hip):
    n = 1 << 22
    t = hip.empty((n,))
    hip.rand_uniform(t, 1.0, 5)
    u = t.numpy().astype(np.float64)
    se = 1.0 / np.sqrt(n)
    assert abs(u.mean() - 0.5) < 5 * np.sqrt(1 / 12.0) * se
    assert abs(u.var() - 1 / 12.0) < 5 * np.sqrt(1 / 180.0) * se
    counts = np.histogram(u, bins=64, range=(0, 1))[0]
    chi2 = ((counts - n / 64.0) ** 2 / (n / 64.0)).sum()
    assert chi2 < 63 + 5 * np.sqrt(2 * 63)                # chi-square with 63 degrees of freedom
    hip.rand_binary(t, 0.25, 6)
    assert abs(t.numpy().mean() - 0.25) < 5 * np.sqrt(0.25 * 0.75) * se


def test_scalar_operations_exact_and_in_place(hip):
    rng = np.random.default_rng(3)
    for n in (1, 5, 4096, 100001):
        x = rng.standard_normal(n, dtype=np.float32)
        a, b = hip.array(x), hip.empty((n,))
        hip.mult_scalar(a, b, 0.3)
        assert np.array_equal(b.numpy(), x * np.float32(0.3))
        hip.add_scalar(a, b, -1.7)
        assert np.array_equal(b.numpy(), x + np.float32(-1.7))
        hip.mult_scalar(a, a, 2.5)   # Tensor::mult_
        hip.add_scalar(a, a, 0.125)  # Tensor::add_
        assert np.array_equal(a.numpy(), x * np.float32(2.5) + np.float32(0.125))


def test_initialiser_recipes(hip):
    """The initialisers of the reference composed from these entry points give the deviations they are named for:
    Glorot uniform (signed uniform x sqrt(6 / (fan_in + fan_out)), src/initializers/initializer_glorot_uniform.cpp:35-60)
    and He normal (normal(0, sqrt(2 / fan_in)), src/initializers/initializer_he_normal.cpp:33-42)."""
    Kf, C, R, S = 256, 128, 3, 3
    n = Kf * C * R * S
    se = 1.0 / np.sqrt(n)
    K = hip.empty((Kf, C, R, S))
    fan_in, fan_out = C * R * S, Kf * R * S
    limit = np.sqrt(6.0 / (fan_in + fan_out))
    hip.rand_signed_uniform(K, 1.0, 21)
    hip.mult_scalar(K, K, limit)
    k = K.numpy().astype(np.float64)
    assert np.abs(k).max() <= np.float32(limit)
    assert abs(k.std() / (limit / np.sqrt(3.0)) - 1.0) < 5 * np.sqrt(0.2) * se * 2  # sd of a uniform variance estimate: sqrt(0.8/n) relative
    assert abs(k.mean()) < 5 * limit / np.sqrt(3.0) * se
    s = np.sqrt(2.0 / fan_in)
    hip.rand_normal(K, 0.0, s, 22)
    k = K.numpy().astype(np.float64)
    assert abs(k.std() / s - 1.0) < 5 * np.sqrt(0.5) * se
    assert abs(k.mean()) < 5 * s * se
    # a registered filter tensor that is re-initialised through these calls is repacked before its next use
    x = hip.array(np.random.default_rng(4).standard_normal((2, C, 8, 8), dtype=np.float32))
    O1, O2 = hip.empty((2, Kf, 8, 8)), hip.empty((2, Kf, 8, 8))
    hip.cache_conv_filters(K)
    hip.conv2D(x, K, None, O1, 1, 1, 1, 1)
    hip.rand_normal(K, 0.0, s, 23)
    hip.conv2D(x, K, None, O1, 1, 1, 1, 1)
    hip.uncache_conv_filters(K)
    hip.conv2D(x, K, None, O2, 1, 1, 1, 1)
    assert np.array_equal(O1.numpy(), O2.numpy())
