"""Seeded input recipe shared by the golden-vector writer and the tests."""

import numpy as np


def inputs(seed, n, m, d, uniform=False, y_shift=0.0, scale=1.0):
    """Shared recipe: tests regenerate the same inputs from (seed, n, m, d)."""
    rng = np.random.default_rng(seed)
    x = (scale * rng.standard_normal((n, d))).astype(np.float32)
    y = (scale * rng.standard_normal((m, d)) + y_shift).astype(np.float32)
    if uniform:
        a = np.full(n, 1.0 / n, np.float32)
        b = np.full(m, 1.0 / m, np.float32)
    else:
        a = rng.random(n).astype(np.float32) + 0.1
        b = rng.random(m).astype(np.float32) + 0.1
        a /= a.sum()
        b /= b.sum()
    return x, y, a, b
