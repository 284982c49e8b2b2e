"""Seeded tensor generator (ngraph/testing/random.py:21-155)."""
import numpy as np


class RandomTensorGenerator(object):
    def __init__(self, seed=0, dtype=np.float32):
        self.dtype = dtype
        self.reset(seed)

    def reset(self, seed=0):
        self.seed = seed
        self.rng = np.random.RandomState(seed=seed)

    def uniform(self, low, high, axes, dtype=None):
        dtype = dtype or self.dtype
        return np.array(self.rng.uniform(low, high, axes.lengths), dtype=dtype)

    def normal(self, loc, scale, axes, dtype=None):
        dtype = dtype or self.dtype
        return np.array(self.rng.normal(loc, scale, axes.lengths), dtype=dtype)

    def discrete_uniform(self, low, high, quantum, axes, dtype=None):
        dtype = dtype or self.dtype
        n = int(round((high - low) / quantum))
        return np.array(self.rng.randint(0, n + 1, axes.lengths) * quantum + low, dtype=dtype)

    def random_integers(self, low, high, axes, dtype=np.int8):
        return self.rng.randint(low, high + 1, axes.lengths).astype(dtype)
