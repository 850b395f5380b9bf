"""TurboQuant = PolarQuant at b-1 bits + 1-bit QJL on the residual, and the
MSE-only variant, with the reference's interface (turboquant/turboquant.py:33-171)."""
from __future__ import annotations

from dataclasses import dataclass

import numpy as np

from .polar_quant import PolarQuant
from .qjl import QJL


@dataclass
class CompressedVector:
    """turboquant/turboquant.py:33-40."""
    mse_indices: np.ndarray     # (d,) or (batch, d), (b-1)-bit codebook indices
    vector_norms: np.ndarray    # scalar or (batch,), ||x||
    qjl_signs: np.ndarray       # (d,) or (batch, d), int8 {+1,-1}
    residual_norms: np.ndarray  # scalar or (batch,), ||x - x_mse||
    bit_width: int              # total bits per coordinate


class TurboQuant:
    def __init__(self, d: int, bit_width: int, seed: int = 42, norm_correction: bool = True, *,
                 rotation: str = "dense", projection: str = "orthogonal"):
        if bit_width < 2:
            raise ValueError("TurboQuant requires bit_width >= 2 (1 bit PolarQuant + 1 bit QJL). "
                             "For 1-bit, use QJL directly.")
        self.d = d
        self.bit_width = bit_width
        self.polar_quant = PolarQuant(d, bit_width=bit_width - 1, seed=seed, norm_correction=norm_correction,
                                      rotation=rotation)
        self.qjl = QJL(d, seed=seed + 1000, projection=projection)  # turboquant/turboquant.py:77

    def quantize(self, x) -> CompressedVector:
        idx, norms, residual = self.polar_quant.quantize_and_residual(x)
        signs, rnorms = self.qjl.quantize(residual)
        return CompressedVector(mse_indices=idx, vector_norms=norms, qjl_signs=signs, residual_norms=rnorms,
                                bit_width=self.bit_width)

    def dequantize(self, compressed: CompressedVector, shrinkage: float = 1.0):
        return (self.polar_quant.dequantize(compressed.mse_indices, compressed.vector_norms)
                + self.qjl.dequantize(compressed.qjl_signs, compressed.residual_norms, shrinkage=shrinkage))

    def compressed_size_bits(self, n_vectors: int) -> int:
        """b bits per coordinate plus one 32-bit norm per vector (turboquant/turboquant.py:126-136)."""
        return n_vectors * (self.d * self.bit_width + 32)

    def compression_ratio(self, original_bits_per_value: int = 16) -> float:
        return (self.d * original_bits_per_value) / (self.d * self.bit_width + 32)


class TurboQuantMSE:
    """PolarQuant at the full bit width, no QJL stage (turboquant/turboquant.py:152-171)."""

    def __init__(self, d: int, bit_width: int, seed: int = 42, norm_correction: bool = True, *,
                 rotation: str = "dense"):
        self.d = d
        self.bit_width = bit_width
        self.polar_quant = PolarQuant(d, bit_width=bit_width, seed=seed, norm_correction=norm_correction,
                                      rotation=rotation)

    def quantize(self, x):
        return self.polar_quant.quantize(x)

    def dequantize(self, indices, norms):
        return self.polar_quant.dequantize(indices, norms)
