"""KV-cache compressor with the reference's interface (turboquant/kv_cache.py:30-188).

One K quantiser (TurboQuant, seed) and one V quantiser (TurboQuantMSE,
seed + 500) serve every layer and head, so the reference's layers x heads loop
collapses into one kernel launch over all L*H*S vectors; the per-(layer, head)
containers are views of that result.
"""
from __future__ import annotations

from dataclasses import dataclass, field

import numpy as np

from .turboquant import CompressedVector, TurboQuant, TurboQuantMSE


@dataclass
class CompressedKVCache:
    """turboquant/kv_cache.py:30-44."""
    k_compressed: list = field(default_factory=list)   # [layer][head] CompressedVector over seq
    v_indices: list = field(default_factory=list)      # [layer][head] (seq, head_dim)
    v_norms: list = field(default_factory=list)        # [layer][head] (seq,)
    num_layers: int = 0
    num_heads: int = 0
    seq_len: int = 0
    head_dim: int = 0
    k_bit_width: int = 0
    v_bit_width: int = 0


class KVCacheCompressor:
    def __init__(self, head_dim: int, k_bits: int = 3, v_bits: int = 3, seed: int = 42,
                 norm_correction: bool = True):
        self.head_dim = head_dim
        self.k_bits = k_bits
        self.v_bits = v_bits
        self.k_quantizer = TurboQuant(head_dim, bit_width=k_bits, seed=seed, norm_correction=norm_correction)
        self.v_quantizer = TurboQuantMSE(head_dim, bit_width=v_bits, seed=seed + 500,
                                         norm_correction=norm_correction)

    def compress(self, k_cache: np.ndarray, v_cache: np.ndarray) -> CompressedKVCache:
        L, H, S, D = k_cache.shape
        assert D == self.head_dim
        assert v_cache.shape == k_cache.shape
        out = CompressedKVCache(num_layers=L, num_heads=H, seq_len=S, head_dim=D,
                                k_bit_width=self.k_bits, v_bit_width=self.v_bits)
        kc = self.k_quantizer.quantize(np.asarray(k_cache).reshape(L * H * S, D))
        vi, vn = self.v_quantizer.quantize(np.asarray(v_cache).reshape(L * H * S, D))
        k_idx = kc.mse_indices.reshape(L, H, S, D)
        k_nrm = kc.vector_norms.reshape(L, H, S)
        k_sgn = kc.qjl_signs.reshape(L, H, S, D)
        k_rn = kc.residual_norms.reshape(L, H, S)
        vi, vn = vi.reshape(L, H, S, D), vn.reshape(L, H, S)
        for l in range(L):
            out.k_compressed.append([CompressedVector(k_idx[l, h], k_nrm[l, h], k_sgn[l, h], k_rn[l, h], self.k_bits)
                                     for h in range(H)])
            out.v_indices.append([vi[l, h] for h in range(H)])
            out.v_norms.append([vn[l, h] for h in range(H)])
        return out

    def decompress(self, compressed: CompressedKVCache):
        L, H, S, D = compressed.num_layers, compressed.num_heads, compressed.seq_len, compressed.head_dim
        cat = lambda rows: np.concatenate([np.asarray(r).reshape(-1, *np.shape(r)[1:]) for r in rows], axis=0)
        flat = [compressed.k_compressed[l][h] for l in range(L) for h in range(H)]
        if not flat or S == 0:
            z = np.zeros((L, H, S, D))
            return z, z.copy()
        kc = CompressedVector(cat([c.mse_indices for c in flat]), cat([c.vector_norms for c in flat]),
                              cat([c.qjl_signs for c in flat]), cat([c.residual_norms for c in flat]), self.k_bits)
        k = self.k_quantizer.dequantize(kc).reshape(L, H, S, D)
        vi = cat([compressed.v_indices[l][h] for l in range(L) for h in range(H)])
        vn = cat([compressed.v_norms[l][h] for l in range(L) for h in range(H)])
        v = self.v_quantizer.dequantize(vi, vn).reshape(L, H, S, D)
        return k, v

    def memory_stats(self, seq_len: int, num_layers: int, num_heads: int) -> dict:
        """turboquant/kv_cache.py:167-188: K counts b bits + a 32-bit norm, V counts b bits."""
        n = num_layers * num_heads * seq_len
        original = n * self.head_dim * 2
        compressed = (n * (self.head_dim * self.k_bits + 32) + n * self.head_dim * self.v_bits) / 8
        return {
            "original_mb": original / 1024 / 1024,
            "compressed_mb": compressed / 1024 / 1024,
            "compression_ratio": original / compressed,
            "k_bits_per_value": self.k_bits,
            "v_bits_per_value": self.v_bits,
        }
