"""Seeded synthetic datasets of the benchmark configurations (host side, numpy) and the
epsilon calibration used by the tests.  All return FP16 bit patterns (uint16) row-major."""
import numpy as np


def exponential(n, d, lam=40.0, seed=1234):
    """i.i.d. Exp(lambda) clipped to [0, 1], quantised to FP16."""
    rng = np.random.default_rng(seed)
    x = rng.exponential(1.0 / lam, size=(n, d))
    return np.clip(x, 0.0, 1.0).astype(np.float32).astype(np.float16).view(np.uint16)


def uniform_bytes(n, d, seed=1234):
    """uniform integers 0..255 scaled by 1/255."""
    rng = np.random.default_rng(seed)
    x = rng.integers(0, 256, size=(n, d)).astype(np.float64) / 255.0
    return x.astype(np.float32).astype(np.float16).view(np.uint16)


def gaussian_mixture(n, d, clusters=1000, sigma=0.05, seed=1234):
    rng = np.random.default_rng(seed)
    centers = rng.random((clusters, d))
    which = rng.integers(0, clusters, size=n)
    x = centers[which] + sigma * rng.standard_normal((n, d))
    return x.astype(np.float32).astype(np.float16).view(np.uint16)


def unit_normal(n, d, seed=1234):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((n, d)).astype(np.float32)
    x /= np.linalg.norm(x, axis=1, keepdims=True)
    return x.astype(np.float16).view(np.uint16)


def small_integers(n, d, high=4, seed=1234):
    """integer coordinates: every product and partial sum is exact in FP32, so any operand
    layout mistake in the matrix-core path shows up as a hard pair-set mismatch."""
    rng = np.random.default_rng(seed)
    return rng.integers(0, high, size=(n, d)).astype(np.float16).view(np.uint16)


def epsilon_for_neighbours(bits, mean_neighbours, sample=512, seed=99):
    """epsilon from a seeded sample of query rows: the distance quantile that gives the wanted
    mean number of neighbours per point (self excluded)."""
    x = bits.view(np.float16).astype(np.float64)
    n = x.shape[0]
    rng = np.random.default_rng(seed)
    rows = rng.choice(n, size=min(sample, n), replace=False)
    sq = (x * x).sum(1)
    d2 = sq[rows][:, None] + sq[None, :] - 2.0 * (x[rows] @ x.T)
    d2[np.arange(len(rows)), rows] = np.inf
    k = int(round(mean_neighbours * len(rows)))
    flat = np.partition(d2.reshape(-1), k)[: k + 1]
    lo, hi = np.sort(flat)[-2:]
    return float(np.sqrt(max(0.5 * (lo + hi), 0.0)))
