"""Oracle: Lloyd-Max scalar codebooks for one coordinate of a rotated unit vector.

Follows /root/reference/codebook.py:14-113 (``beta_pdf_normalized``,
``lloyd_max_iteration``, ``compute_codebook``) and the fp32 cast in
/root/reference/kvquant/tq_backend.py:39-46.

The reference integrates on a fixed grid of 10,000 points over +-5 sigma and
selects each Voronoi cell with a boolean mask ``(x >= lo) & (x < hi)``.  On a
sorted grid that mask is an index range, so this restatement finds the range
with a binary search and sums the slice; numpy's pairwise summation only depends
on the values and their count, so the sums are the same doubles.
"""
from __future__ import annotations

import math

import numpy as np

N_GRID = 10_000          # codebook.py:40 (n_quad default)
MAX_ITERS = 500          # codebook.py:78
TOL = 1e-10              # codebook.py:79
X_RANGE = 5.0            # codebook.py:80

_SQRT_2PI = np.sqrt(2 * np.pi)


def coordinate_pdf(x: np.ndarray, d: int) -> np.ndarray:
    """Density of one coordinate of a uniform unit vector in R^d (codebook.py:14-33).

    d >= 100: N(0, 1/d), written the way scipy evaluates ``norm.pdf(x, 0, std)``
    (standardise, ``exp(-z*z/2)/sqrt(2 pi)``, divide by the scale).
    d < 100: Beta((d-1)/2, (d-1)/2) mapped to [-1, 1].
    """
    if d >= 100:
        std = 1.0 / np.sqrt(d)
        z = np.asarray((x - 0) / std, dtype=np.float64)
        return np.exp(-z ** 2 / 2.0) / _SQRT_2PI / std
    from scipy import stats  # exact small-d branch only (codebook.py:27-33)
    a = (d - 1) / 2.0
    t = (x + 1) / 2.0
    inside = (x >= -1) & (x <= 1)
    t = np.clip(t, 1e-10, 1 - 1e-10)
    return np.where(inside, stats.beta.pdf(t, a, a) / 2.0, 0.0)


def _lloyd_step(c: np.ndarray, x: np.ndarray, px: np.ndarray, dx: float,
                x_min: float, x_max: float) -> np.ndarray:
    """One conditional-mean update (codebook.py:36-72)."""
    c = np.sort(c)
    edges = np.concatenate([[x_min], (c[:-1] + c[1:]) / 2, [x_max]])
    # first grid index with x >= edge; cell i is the half-open range [cut[i], cut[i+1])
    cut = np.searchsorted(x, edges, side="left")
    out = np.zeros(len(c))
    for i in range(len(c)):
        a, b = cut[i], cut[i + 1]
        w = px[a:b]
        mass = np.sum(w) * dx
        out[i] = np.sum(x[a:b] * w) * dx / mass if mass > 0 else c[i]
    return out


def lloyd_max_codebook(k: int, d: int) -> np.ndarray:
    """Sorted fp64 centroids, ``k`` levels, dimension ``d`` (codebook.py:75-113)."""
    std = 1.0 / np.sqrt(d)
    if d < 100:
        x_min, x_max = -1.0, 1.0
    else:
        x_min, x_max = -X_RANGE * std, X_RANGE * std
    x = np.linspace(x_min, x_max, N_GRID)
    dx = x[1] - x[0]
    px = coordinate_pdf(x, d)
    c = np.linspace(-3 * std, 3 * std, k)
    new = c
    for _ in range(MAX_ITERS):
        new = _lloyd_step(c, x, px, dx, x_min, x_max)
        if np.max(np.abs(new - c)) < TOL:
            break          # the fresh iterate is what gets returned (codebook.py:107-113)
        c = new
    return np.sort(new)


_CACHE: dict[tuple[int, int], np.ndarray] = {}


def codebook_f32(bits: int, d: int) -> np.ndarray:
    """fp32 table of 2**bits centroids, cached per (bits, d) (tq_backend.py:39-46)."""
    key = (bits, d)
    if key not in _CACHE:
        _CACHE[key] = lloyd_max_codebook(2 ** bits, d).astype(np.float32)
    return _CACHE[key]


def distortion(c: np.ndarray, d: int, n_grid: int = 20_000) -> float:
    """Per-coordinate MSE of codebook ``c`` (codebook.py:116-143), used by tests."""
    std = 1.0 / math.sqrt(d)
    lo, hi = (-1.0, 1.0) if d < 100 else (-X_RANGE * std, X_RANGE * std)
    x = np.linspace(lo, hi, n_grid)
    dx = x[1] - x[0]
    px = coordinate_pdf(x, d)
    edges = np.concatenate([[lo], (c[:-1] + c[1:]) / 2, [hi]])
    cut = np.searchsorted(x, edges, side="left")
    total = 0.0
    for i in range(len(c)):
        a, b = cut[i], cut[i + 1]
        total += np.sum((x[a:b] - c[i]) ** 2 * px[a:b]) * dx
    return float(total)
