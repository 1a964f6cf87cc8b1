"""Comparison helpers shared by the parity tests."""
import numpy as np


def kept_mask(offsets, K):
    """Boolean mask over the fragment buffer: entry belongs to the first min(count, K) of its pixel list."""
    offsets = np.asarray(offsets, dtype=np.int64)
    counts = np.diff(offsets)
    total = int(offsets[-1])
    rank = np.arange(total, dtype=np.int64) - np.repeat(offsets[:-1], counts)
    if K is None or K <= 0:
        return np.ones(total, dtype=bool)
    return rank < K


def rel_err(a, b, floor_frac=1e-3):
    """Element-wise |a-b| / max(|b|, floor) with floor = floor_frac * max|b| (guards elements that cancel to ~0)."""
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    scale = float(np.max(np.abs(b))) if b.size else 0.0
    floor = max(scale * floor_frac, 1e-30)
    return np.abs(a - b) / np.maximum(np.abs(b), floor)


def max_rel_err(a, b, floor_frac=1e-3):
    e = rel_err(a, b, floor_frac)
    return float(e.max()) if e.size else 0.0
