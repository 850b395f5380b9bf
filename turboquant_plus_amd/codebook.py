"""Lloyd-Max codebooks for the post-rotation coordinate distribution
(turboquant/codebook.py:29-134).

The codebook is a one-off host-side table (SciPy normal cdf/pdf/ppf, exactly
100 Lloyd rounds: the iteration count is part of parity); looking values up in
it runs on the GPU.
"""
from __future__ import annotations

import numpy as np
from scipy import stats

from . import _lib as L


def _gaussian_conditional_expectation(sigma: float, a: float, b: float) -> float:
    """E[X | a < X < b] for X ~ N(0, sigma^2) (turboquant/codebook.py:88-118),
    including its fallbacks when the interval holds less than 1e-15 mass."""
    lo = a / sigma if np.isfinite(a) else a
    hi = b / sigma if np.isfinite(b) else b
    if not np.isfinite(lo):
        mass = stats.norm.cdf(hi)
    elif not np.isfinite(hi):
        mass = stats.norm.sf(lo)
    else:
        mass = stats.norm.cdf(hi) - stats.norm.cdf(lo)
    if mass < 1e-15:
        if np.isfinite(a) and not np.isfinite(b):
            return a + sigma
        if np.isfinite(b) and not np.isfinite(a):
            return b - sigma
        if np.isfinite(a) and np.isfinite(b):
            return (a + b) / 2.0
        return 0.0
    return sigma * (stats.norm.pdf(lo) - stats.norm.pdf(hi)) / mass


def _lloyds_gaussian(n_centroids: int, sigma: float, n_iter: int = 100) -> np.ndarray:
    """Lloyd iteration from equiprobable cells (turboquant/codebook.py:52-85)."""
    cuts = stats.norm.ppf(np.linspace(0, 1, n_centroids + 1)[1:-1], scale=sigma)
    levels = np.zeros(n_centroids)
    for round_ in range(n_iter + 1):
        if round_:
            cuts = (levels[:-1] + levels[1:]) / 2.0
        edges = np.concatenate(([-np.inf], cuts, [np.inf]))
        for i in range(n_centroids):
            levels[i] = _gaussian_conditional_expectation(sigma, edges[i], edges[i + 1])
    return np.sort(levels)


def optimal_centroids(bit_width: int, d: int) -> np.ndarray:
    """Sorted 2^bit_width centroids for N(0, 1/d) (turboquant/codebook.py:29-49)."""
    if bit_width == 1:
        c = np.sqrt(2.0 / (np.pi * d))
        return np.array([-c, c])
    if bit_width == 2:
        return np.array([-1.51, -0.453, 0.453, 1.51]) / np.sqrt(d)
    return _lloyds_gaussian(1 << bit_width, sigma=1.0 / np.sqrt(d))


def nearest_centroid_indices(values: np.ndarray, centroids: np.ndarray) -> np.ndarray:
    """Index of the nearest centroid = number of midpoints strictly below the
    value, ties to the lower index (turboquant/codebook.py:121-134); GPU kernel."""
    values = np.asarray(values)
    centroids = np.ascontiguousarray(centroids, dtype=np.float64)
    if len(centroids) > 256:
        raise NotImplementedError("at most 256 centroids")
    tt = L.torch()
    vd = L.to_device(values.astype(np.float64).ravel())
    out = tt.empty(vd.numel(), dtype=tt.int32, device=vd.device)
    L.check(L.lib().tq_nearest_centroid(L.ptr(vd), vd.numel(), L.dbl_ptr(centroids), len(centroids), L.ptr(out),
                                        L.stream_ptr()))
    return out.cpu().numpy().astype(np.intp).reshape(values.shape)
