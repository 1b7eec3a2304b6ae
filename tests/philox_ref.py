"""Philox4x32-10 in numpy (Salmon, Moraes, Dror, Shaw, "Parallel random numbers: as easy as 1, 2, 3", SC'11), written
from the paper's round function, as the checker of the device generator behind eddlhip_rand_*.  It is pinned itself
by the known-answer vectors that the algorithm's authors publish with their Random123 library (kat_vectors,
philox4x32 with 10 rounds), see test_generator_cpu.py.

Not a restatement of anything in the reference: EDDL draws from cuRAND / std::mt19937, whose streams are not part
of its contract (and are seeded from std::random_device on the CPU).
"""
import numpy as np

M0, M1 = np.uint64(0xD2511F53), np.uint64(0xCD9E8D57)
W0, W1 = 0x9E3779B9, 0xBB67AE85
MASK = np.uint64(0xFFFFFFFF)


def philox4x32_10(counter, key):
    """counter: uint32 array [..., 4]; key: (k0, k1).  Returns uint32 array [..., 4]."""
    c = [np.asarray(counter[..., j], dtype=np.uint64) for j in range(4)]
    k0, k1 = int(key[0]), int(key[1])
    for _ in range(10):
        p0 = M0 * c[0]
        p1 = M1 * c[2]
        hi0, lo0 = p0 >> np.uint64(32), p0 & MASK
        hi1, lo1 = p1 >> np.uint64(32), p1 & MASK
        c = [hi1 ^ c[1] ^ np.uint64(k0), lo1, hi0 ^ c[3] ^ np.uint64(k1), lo0]
        k0 = (k0 + W0) & 0xFFFFFFFF
        k1 = (k1 + W1) & 0xFFFFFFFF
    return np.stack(c, axis=-1).astype(np.uint32)


def words(n, seed, first_block=0, counter_hi=0):
    """The first n words of the stream eddlhip_rand_words(seed, first_block, counter_hi) writes."""
    nb = (n + 3) // 4
    b = (np.arange(nb, dtype=np.uint64) + np.uint64(first_block & 0xFFFFFFFFFFFFFFFF))  # wraps modulo 2^64
    ctr = np.empty((nb, 4), np.uint32)
    ctr[:, 0] = (b & MASK).astype(np.uint32)
    ctr[:, 1] = (b >> np.uint64(32)).astype(np.uint32)
    ctr[:, 2] = counter_hi & 0xFFFFFFFF
    ctr[:, 3] = (counter_hi >> 32) & 0xFFFFFFFF
    return philox4x32_10(ctr, (seed & 0xFFFFFFFF, (seed >> 32) & 0xFFFFFFFF)).reshape(-1)[:n]


UNIFORM, SIGNED_UNIFORM, BINARY, NORMAL = 0, 1, 2, 3  # third counter word of the four kinds of fill


def unit(w):
    return (w >> np.uint32(8)).astype(np.float32) * np.float32(2.0 ** -24)


def uniform(n, v, seed):
    return unit(words(n, seed, 0, UNIFORM)) * np.float32(v)


def signed_uniform(n, v, seed):
    return (np.float32(2.0) * unit(words(n, seed, 0, SIGNED_UNIFORM)) - np.float32(1.0)) * np.float32(v)


def binary(n, v, seed):
    return (unit(words(n, seed, 0, BINARY)) < np.float32(v)).astype(np.float32)


def normal(n, mean, stddev, seed):
    """Box-Muller in float64 from the same words the device uses: words (0, 1) of a block give elements 0 and 1
    (cosine and sine branch), words (2, 3) elements 2 and 3."""
    w = words(4 * ((n + 3) // 4), seed, 0, NORMAL).reshape(-1, 2, 2)
    u1 = ((w[..., 0] >> np.uint32(8)).astype(np.float64) + 1.0) * 2.0 ** -24
    u2 = (w[..., 1] >> np.uint32(8)).astype(np.float64) * 2.0 ** -24
    r = np.sqrt(-2.0 * np.log(u1))
    z = np.stack([r * np.cos(2 * np.pi * u2), r * np.sin(2 * np.pi * u2)], axis=-1)
    return (z.reshape(-1)[:n] * stddev + mean)
