"""QJL 1-bit sign sketch with the reference's interface (turboquant/qjl.py:32-134).

`projection="orthogonal"` (default) is the reference class: QR-orthogonalised
Gaussian, reconstruction scale sqrt(pi/2)/sqrt(d).  `projection="gaussian"`
keeps the raw Gaussian matrix with scale sqrt(pi/2)/d (the paper's form).
The projections run as float64 HIP kernels (tq_qjl_quantize / tq_qjl_dequantize).
"""
from __future__ import annotations

import numpy as np

from . import _lib as L

QJL_CONST = np.sqrt(np.pi / 2)


def projection_matrix(d: int, seed: int, projection: str = "orthogonal"):
    """(S, scale) for a seed (turboquant/qjl.py:57-62)."""
    g = np.random.default_rng(seed).standard_normal((d, d))
    if projection == "gaussian":
        return g, QJL_CONST / d
    if projection != "orthogonal":
        raise ValueError(f"projection must be 'orthogonal' or 'gaussian', got {projection!r}")
    q, r = np.linalg.qr(g)
    return q * np.sign(np.diag(r))[None, :], QJL_CONST / np.sqrt(d)


class QJL:
    _ORTHO_TOL = 1e-10

    def __init__(self, d: int, seed: int = 123, *, projection: str = "orthogonal"):
        self.d = d
        self.projection = projection
        self.S, self.scale = projection_matrix(d, seed, projection)
        if projection == "orthogonal":
            err = np.linalg.norm(self.S @ self.S.T - np.eye(d), "fro")
            assert err < self._ORTHO_TOL, f"QJL projection matrix not orthogonal: ||S S^T - I||_F = {err:.2e}"
        self._handle = None

    @property
    def handle(self) -> L.Handle:
        if self._handle is None:
            self._handle = L.Handle(self.d, 1, np.array([-1.0, 1.0]), rotation=np.eye(self.d), projection=self.S,
                                    projection_scale=self.scale)
        return self._handle

    def quantize(self, r):
        """(signs int8 in {+1,-1}, norms float64) (turboquant/qjl.py:72-94)."""
        r = np.asarray(r)
        single = r.ndim == 1
        r2 = r[None, :] if single else r
        if r2.shape[-1] != self.d:
            raise ValueError(f"quantize: last dimension must be {self.d}")
        tt = L.torch()
        rd = L.to_device(r2)
        n = rd.shape[0]
        signs = tt.empty((n, self.d), dtype=tt.int8, device=rd.device)
        norms = tt.empty((n,), dtype=tt.float64, device=rd.device)
        L.check(L.lib().tq_qjl_quantize(self.handle.h, L.ptr(rd), n, L.dtype_code(rd), L.ptr(signs), L.ptr(norms),
                                        L.stream_ptr()))
        s, nn = signs.cpu().numpy(), norms.cpu().numpy()
        return (s[0], nn[0]) if single else (s, nn)

    def dequantize(self, signs, norms, shrinkage: float = 1.0):
        """scale * norm * shrinkage * S^T signs (turboquant/qjl.py:96-134)."""
        signs = np.asarray(signs)
        single = signs.ndim == 1
        if single:
            signs = signs[None, :]
            norms = np.array([norms])
        tt = L.torch()
        dev = L.require_gpu()
        sd = tt.from_numpy(np.ascontiguousarray(signs, dtype=np.int8)).to(dev)
        nd = tt.from_numpy(np.ascontiguousarray(np.asarray(norms, dtype=np.float64).reshape(-1))).to(dev)
        n = sd.shape[0]
        out = tt.empty((n, self.d), dtype=tt.float64, device=dev)
        L.check(L.lib().tq_qjl_dequantize(self.handle.h, L.ptr(sd), L.ptr(nd), float(shrinkage), n, L.ptr(out),
                                          L.stream_ptr()))
        res = out.cpu().numpy()
        return res[0] if single else res
