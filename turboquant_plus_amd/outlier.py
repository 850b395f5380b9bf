"""Fractional bit rates by splitting the channels between two PolarQuant
instances of neighbouring widths, with one QJL sketch over the full residual
(interface of turboquant/outlier.py:33-217).  The per-vector arithmetic runs
in the PolarQuant / QJL kernels; this module only routes channels."""
from __future__ import annotations

from dataclasses import dataclass

import numpy as np

from .polar_quant import PolarQuant
from .qjl import QJL


@dataclass
class OutlierCompressedVector:
    """turboquant/outlier.py:33-42."""
    outlier_indices: np.ndarray
    outlier_norms: np.ndarray
    normal_indices: np.ndarray
    normal_norms: np.ndarray
    qjl_signs: np.ndarray
    residual_norms: np.ndarray
    effective_bits: float


def _compute_channel_split(d: int, target_bits: float) -> tuple[int, int, int, int]:
    """(n_outlier, outlier_bits, n_normal, normal_bits), turboquant/outlier.py:45-67."""
    low_bits = int(np.floor(target_bits))
    n_outlier = int(round(d * (target_bits - low_bits)))
    return n_outlier, low_bits + 1, d - n_outlier, low_bits


class OutlierTurboQuant:
    def __init__(self, d: int, target_bits: float, seed: int = 42):
        self.d = d
        self.target_bits = target_bits
        self.n_outlier, self.high_bits, self.n_normal, self.low_bits = _compute_channel_split(d, target_bits)
        self.effective_bits = (self.n_outlier * self.high_bits + self.n_normal * self.low_bits) / d
        self.outlier_idx = np.arange(self.n_outlier)           # fixed split: the first n_outlier channels
        self.normal_idx = np.arange(self.n_outlier, d)
        self.pq_outlier = (PolarQuant(self.n_outlier, bit_width=self.high_bits - 1, seed=seed)
                           if self.n_outlier > 0 else None)
        self.pq_normal = (PolarQuant(self.n_normal, bit_width=self.low_bits - 1, seed=seed + 500)
                          if self.n_normal > 0 else None)
        self.qjl = QJL(d, seed=seed + 1000)

    def quantize(self, x) -> OutlierCompressedVector:
        x = np.asarray(x)
        single = x.ndim == 1
        xb = x[np.newaxis, :] if single else x
        batch = xb.shape[0]
        residual = np.zeros((batch, self.d))
        parts = []
        for pq, cols in ((self.pq_outlier, self.outlier_idx), (self.pq_normal, self.normal_idx)):
            if pq is None:
                parts += [np.array([]), np.array([])]
                continue
            sub = np.ascontiguousarray(xb[:, cols])
            # a batch of one goes through the single-vector path (turboquant/outlier.py:124,132)
            idx, norms, res = pq.quantize_and_residual(sub if batch > 1 else sub[0])
            residual[:, cols] = res
            parts += [idx, norms]
        signs, rnorms = self.qjl.quantize(residual[0] if single else residual)
        return OutlierCompressedVector(outlier_indices=parts[0], outlier_norms=parts[1], normal_indices=parts[2],
                                       normal_norms=parts[3], qjl_signs=signs, residual_norms=rnorms,
                                       effective_bits=self.effective_bits)

    def dequantize(self, compressed: OutlierCompressedVector) -> np.ndarray:
        x_hat = self.qjl.dequantize(compressed.qjl_signs, compressed.residual_norms)
        x_hat = np.array(x_hat, dtype=np.float64)
        if self.pq_outlier is not None:
            x_hat[..., self.outlier_idx] += self.pq_outlier.dequantize(compressed.outlier_indices,
                                                                       compressed.outlier_norms)
        if self.pq_normal is not None:
            x_hat[..., self.normal_idx] += self.pq_normal.dequantize(compressed.normal_indices,
                                                                     compressed.normal_norms)
        return x_hat

    def compression_ratio(self, original_bits: int = 16) -> float:
        """d * effective_bits + one 32-bit residual norm + two 32-bit vector norms (turboquant/outlier.py:209-217)."""
        return (self.d * original_bits) / (self.d * self.effective_bits + 32 + 64)
