"""Seeded synthetic inputs for the five benchmark configurations.

Every generator is a pure function of (size, seed) built on numpy's PCG64 stream, so the
parity tests, the CPU baseline and the GPU benchmark all see the same data.
"""
from __future__ import annotations

import numpy as np


def uniform_f32(n, seed, lo=-1.0, hi=1.0):
    """i.i.d. uniform [lo, hi) Float32 (dotp: [-1, 1); scanl1 f32 and Jacobi: [0, 1))."""
    rng = np.random.default_rng(seed)
    return (rng.random(n, dtype=np.float32) * np.float32(hi - lo) + np.float32(lo)).astype(np.float32)


def uniform_int(n, seed, lo=-1000, hi=1000, dtype=np.int64):
    """Uniform integers in [lo, hi] (inclusive)."""
    rng = np.random.default_rng(seed)
    return rng.integers(lo, hi + 1, n, dtype=np.int64).astype(dtype)


def segment_lengths(nseg, total, seed):
    """Segment lengths for the segmented-sum configuration: 90% of the segments draw a length
    uniform in [1, 64], 10% a geometric length with mean 4096; the lengths are then scaled
    to sum to exactly `total` (largest-remainder rounding, so every length stays >= 0 and
    short segments may round to 0, i.e. empty segments occur).  Returns int32[nseg]."""
    rng = np.random.default_rng(seed)
    short = rng.integers(1, 65, nseg, dtype=np.int64)
    long_ = rng.geometric(1.0 / 4096.0, nseg).astype(np.int64)
    pick = rng.random(nseg) < 0.1
    raw = np.where(pick, long_, short).astype(np.float64)
    scaled = raw * (float(total) / raw.sum())
    base = np.floor(scaled).astype(np.int64)
    rem = int(total - base.sum())
    if rem > 0:
        order = np.argsort(-(scaled - base), kind="stable")[:rem]
        base[order] += 1
    assert base.sum() == total and base.min() >= 0
    return base.astype(np.int32)


def zipf_keys(n, nbins, seed, s=1.1):
    """Keys drawn from Zipf(s) over nbins bins by inverse CDF on a seeded uniform; rank r maps
    to bin r (the hottest bin is bin 0).  Returns int32[n]."""
    rng = np.random.default_rng(seed)
    w = np.arange(1, nbins + 1, dtype=np.float64) ** (-s)
    cdf = np.cumsum(w)
    cdf /= cdf[-1]
    u = rng.random(n)
    return np.minimum(np.searchsorted(cdf, u, side="right"), nbins - 1).astype(np.int32)
