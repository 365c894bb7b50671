"""Seeded synthetic inputs shared by the parity tests, the smoke test and the
benchmark (numpy PCG64 streams; nothing is read from disk)."""
import numpy as np


def normal_with_outliers(n, seed, dist="normal", frac=1e-4, mag=50.0):
    """N(0,1) or Laplace(0,1) with `frac` of the positions set to +-mag."""
    rng = np.random.default_rng(seed)
    if dist == "normal":
        x = rng.standard_normal(n, dtype=np.float32)
    elif dist == "laplace":
        x = rng.laplace(0.0, 1.0, n).astype(np.float32)
    else:
        raise ValueError(dist)
    k = max(1, int(round(n * frac))) if n else 0
    if k:
        idx = rng.choice(n, size=k, replace=False)
        x[idx] = mag * rng.choice(np.array([-1.0, 1.0], np.float32), size=k)
    return x


def int32_uniform(n, seed, bits=28):
    rng = np.random.default_rng(seed)
    return rng.integers(-(1 << bits), 1 << bits, size=n, dtype=np.int32)


def int8_uniform(shape, seed, lo=-127, hi=127):
    rng = np.random.default_rng(seed)
    return rng.integers(lo, hi + 1, size=shape, dtype=np.int8)
