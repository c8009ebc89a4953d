"""Shared helpers for the test-suite: seeded inputs and conversions."""
import random

import numpy as np

from pyfield import E2, P


class SplitMix64:
    """Seeded generator used for every synthetic input, so that the same bytes
    reach the GPU library and the checker."""

    def __init__(self, seed):
        self.s = seed & 0xFFFFFFFFFFFFFFFF

    def next(self):
        self.s = (self.s + 0x9E3779B97F4A7C15) & 0xFFFFFFFFFFFFFFFF
        z = self.s
        z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & 0xFFFFFFFFFFFFFFFF
        z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & 0xFFFFFFFFFFFFFFFF
        return z ^ (z >> 31)

    def field(self):
        while True:
            v = self.next()
            if v < P:
                return v


def rand_base(n, seed):
    """n uniform canonical Goldilocks elements (vectorised; rejection is replaced by
    a reduction since the rejected band is 2^-32 wide and tests only need determinism)."""
    rng = np.random.Generator(np.random.PCG64(seed))
    v = rng.integers(0, 2**64, size=n, dtype=np.uint64)
    return np.where(v >= np.uint64(P), v - np.uint64(P), v)


def rand_e2(n, seed):
    return np.stack([rand_base(n, seed * 2 + 1), rand_base(n, seed * 2 + 2)], axis=-1)


def rand_i64(shape, seed, lo=-2048, hi=2047):
    rng = np.random.Generator(np.random.PCG64(seed))
    return rng.integers(lo, hi + 1, size=shape, dtype=np.int64)


def to_E2(arr):
    arr = np.asarray(arr, dtype=np.uint64).reshape(-1, 2)
    return [E2(int(a), int(b)) for a, b in arr]


def from_E2(xs):
    return np.array([[x.a, x.b] for x in xs], dtype=np.uint64).reshape(-1, 2)


def py_rng(seed):
    return random.Random(seed)
