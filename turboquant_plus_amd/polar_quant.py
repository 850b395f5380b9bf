"""PolarQuant with the reference's interface (turboquant/polar_quant.py:46-132):
norm extraction, rotation, nearest Lloyd-Max centroid per coordinate.

Tables are built on the host exactly as the reference builds them; quantize,
dequantize and the residual run as float64 HIP kernels (tq_quantize_indices,
tq_dequantize_indices).  `rotation="wht"` replaces the dense Haar rotation by
the sign-diagonal Walsh-Hadamard rotation D2 H D1 (signs drawn from the same
seeded generator as turboquant/rotation.py:94-95).
"""
from __future__ import annotations

import numpy as np

from . import _lib as L
from .codebook import optimal_centroids
from .rotation import random_rotation_dense, random_rotation_fast


class PolarQuant:
    def __init__(self, d: int, bit_width: int, seed: int = 42, norm_correction: bool = True, *,
                 rotation: str = "dense"):
        if rotation not in ("dense", "wht"):
            raise ValueError(f"rotation must be 'dense' or 'wht', got {rotation!r}")
        if not 1 <= bit_width <= 8:
            raise ValueError(f"bit_width must be 1-8, got {bit_width}")
        self.d = d
        self.bit_width = bit_width
        self.n_centroids = 1 << bit_width
        self.norm_correction = norm_correction
        self.rotation_mode = rotation
        rng = np.random.default_rng(seed)
        if rotation == "dense":
            self.rotation = random_rotation_dense(d, rng)
            self.signs1 = self.signs2 = None
        else:
            self.signs1, self.signs2, self.padded_d = random_rotation_fast(d, rng)
            self.rotation = None
        self.centroids = optimal_centroids(bit_width, d)
        self._handle = None

    # the device tables are created on first use so that constructing a
    # quantiser (and reading .rotation / .centroids) needs no GPU
    @property
    def handle(self) -> L.Handle:
        if self._handle is None:
            self._handle = L.Handle(self.d, self.bit_width, self.centroids, signs1=self.signs1, signs2=self.signs2,
                                    rotation=self.rotation, norm_correction=self.norm_correction)
        return self._handle

    def _check(self, a, what):
        if a.shape[-1] != self.d:
            raise ValueError(f"{what}: last dimension must be {self.d}, got {a.shape[-1]}")

    def quantize(self, x):
        """(indices int64, norms float64); 1-D input gives 1-D indices and a
        scalar norm (turboquant/polar_quant.py:56-85)."""
        x = np.asarray(x)
        single = x.ndim == 1
        x2 = x[None, :] if single else x
        self._check(x2, "quantize")
        tt = L.torch()
        xd = L.to_device(x2)
        n = xd.shape[0]
        idx = tt.empty((n, self.d), dtype=tt.uint8, device=xd.device)
        norms = tt.empty((n,), dtype=tt.float64, device=xd.device)
        L.check(L.lib().tq_quantize_indices(self.handle.h, L.ptr(xd), n, L.dtype_code(xd), L.ptr(idx), L.ptr(norms),
                                            None, L.stream_ptr()))
        idx_h = idx.cpu().numpy().astype(np.int64)
        norms_h = norms.cpu().numpy()
        return (idx_h[0], norms_h[0]) if single else (idx_h, norms_h)

    def _dequantize_device(self, indices, norms, x=None):
        tt = L.torch()
        dev = L.require_gpu()
        idx = tt.from_numpy(np.ascontiguousarray(indices, dtype=np.uint8)).to(dev)
        nd = tt.from_numpy(np.ascontiguousarray(norms, dtype=np.float64)).to(dev)
        n = idx.shape[0]
        out = tt.empty((n, self.d), dtype=tt.float64, device=dev)
        res = xd = None
        if x is not None:
            xd = L.to_device(x)
            res = tt.empty_like(out)
        L.check(L.lib().tq_dequantize_indices(self.handle.h, L.ptr(idx), L.ptr(nd), n, L.ptr(out), L.ptr(xd),
                                              L.dtype_code(xd) if xd is not None else L.TQ_F64, L.ptr(res),
                                              L.stream_ptr()))
        return out.cpu().numpy(), (res.cpu().numpy() if res is not None else None)

    def dequantize(self, indices, norms):
        """Reconstruction, float64 (turboquant/polar_quant.py:87-119)."""
        indices = np.asarray(indices)
        single = indices.ndim == 1
        if single:
            indices = indices[None, :]
            norms = np.array([norms])
        self._check(indices, "dequantize")
        if indices.size and (indices.min() < 0 or indices.max() >= self.n_centroids):
            raise ValueError("indices out of range for this codebook")
        out, _ = self._dequantize_device(indices, np.asarray(norms, dtype=np.float64).reshape(-1))
        return out[0] if single else out

    def quantize_and_residual(self, x):
        """(indices, norms, x - dequantize(indices, norms)) (turboquant/polar_quant.py:121-132)."""
        x = np.asarray(x)
        single = x.ndim == 1
        idx, norms = self.quantize(x)
        x2 = x[None, :] if single else x
        i2 = idx[None, :] if single else idx
        n2 = np.array([norms]) if single else norms
        _, res = self._dequantize_device(i2, n2, x=x2)
        return idx, norms, (res[0] if single else res)
