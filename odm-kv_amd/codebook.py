"""Lloyd-Max codebooks for the coordinates of a randomly rotated unit vector.

Same call as the reference's top-level ``codebook`` module (codebook.py:75-113):
``compute_codebook(k, d)`` returns the sorted fp64 centroids of the k-level scalar quantiser
that minimises squared error under the coordinate density (N(0, 1/d) for d >= 100, the exact
Beta((d-1)/2, (d-1)/2) law on [-1, 1] below that).  The tables are tiny and built once per
(k, d) on the host; the kernels receive them as fp32 arrays.
"""
from __future__ import annotations

import numpy as np

_GRID = 10_000


def _density(x: np.ndarray, d: int) -> np.ndarray:
    if d >= 100:
        scale = 1.0 / np.sqrt(d)
        z = (x - 0) / scale
        return np.exp(-z ** 2 / 2.0) / np.sqrt(2 * np.pi) / scale
    from scipy import stats
    half = (d - 1) / 2.0
    t = np.clip((x + 1) / 2.0, 1e-10, 1 - 1e-10)
    return np.where((x >= -1) & (x <= 1), stats.beta.pdf(t, half, half) / 2.0, 0.0)


def compute_codebook(k: int, d: int, n_iter: int = 500, tol: float = 1e-10,
                     x_range: float = 5.0) -> np.ndarray:
    scale = 1.0 / np.sqrt(d)
    lo, hi = (-1.0, 1.0) if d < 100 else (-x_range * scale, x_range * scale)
    grid = np.linspace(lo, hi, _GRID)
    step = grid[1] - grid[0]
    w = _density(grid, d)
    cur = np.linspace(-3 * scale, 3 * scale, k)
    nxt = cur
    for _ in range(n_iter):
        cur = np.sort(cur)
        walls = np.concatenate([[lo], (cur[:-1] + cur[1:]) / 2, [hi]])
        # cell i = grid points in [walls[i], walls[i+1]); on a sorted grid that is an index range
        idx = np.searchsorted(grid, walls, side="left")
        nxt = np.empty(k)
        for i in range(k):
            a, b = idx[i], idx[i + 1]
            mass = np.sum(w[a:b]) * step
            nxt[i] = np.sum(grid[a:b] * w[a:b]) * step / mass if mass > 0 else cur[i]
        if np.max(np.abs(nxt - cur)) < tol:
            break
        cur = nxt
    return np.sort(nxt)
