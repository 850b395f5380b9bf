"""Host bit-packing formats and footprint arithmetic with the reference's names
(turboquant/utils.py:20-123).  The byte formats are the reference's (MSB-first
streams); the packing itself runs on the GPU.  The device KV layout is a
different, block-structured format (see turbo.py)."""
from __future__ import annotations

import numpy as np

from . import _lib as L


def pack_bits(signs: np.ndarray) -> np.ndarray:
    """{+1,-1} int8 -> bitfield, 8 per byte, first sign in the MSB, rows padded
    to whole bytes (turboquant/utils.py:20-49)."""
    signs = np.asarray(signs)
    single = signs.ndim == 1
    s2 = np.ascontiguousarray(signs.reshape(1, -1) if single else signs).astype(np.int8)
    n, d = s2.shape
    tt = L.torch()
    dev = L.require_gpu()
    sd = tt.from_numpy(s2).to(dev)
    out = tt.empty((n, (d + 7) // 8), dtype=tt.uint8, device=dev)
    L.check(L.lib().tq_pack_bits(L.ptr(sd), n, d, L.ptr(out), L.stream_ptr()))
    res = out.cpu().numpy()
    return res[0] if single else res


def unpack_bits(packed: np.ndarray, d: int) -> np.ndarray:
    """Inverse of pack_bits -> int8 {+1,-1} (turboquant/utils.py:52-68)."""
    packed = np.asarray(packed, dtype=np.uint8)
    single = packed.ndim == 1
    p2 = np.ascontiguousarray(packed.reshape(1, -1) if single else packed)
    n = p2.shape[0]
    if p2.shape[1] != (d + 7) // 8:
        raise ValueError(f"packed rows must hold ceil({d}/8) bytes")
    tt = L.torch()
    dev = L.require_gpu()
    pd_ = tt.from_numpy(p2).to(dev)
    out = tt.empty((n, d), dtype=tt.int8, device=dev)
    L.check(L.lib().tq_unpack_bits(L.ptr(pd_), n, d, L.ptr(out), L.stream_ptr()))
    res = out.cpu().numpy()
    return res[0] if single else res


def pack_indices(indices: np.ndarray, bit_width: int) -> np.ndarray:
    """b-bit indices -> one MSB-first bit stream over the flattened array for
    b <= 4, one byte per index above (turboquant/utils.py:71-98)."""
    if bit_width <= 0 or bit_width > 8:
        raise ValueError(f"bit_width must be 1-8, got {bit_width}")
    indices = np.asarray(indices)
    if bit_width > 4:
        return indices.astype(np.uint8)
    flat = np.ascontiguousarray(indices.ravel().astype(np.uint8))
    tt = L.torch()
    dev = L.require_gpu()
    fd = tt.from_numpy(flat).to(dev)
    out = tt.empty(((flat.size * bit_width + 7) // 8,), dtype=tt.uint8, device=dev)
    L.check(L.lib().tq_pack_indices(L.ptr(fd), flat.size, bit_width, L.ptr(out), L.stream_ptr()))
    return out.cpu().numpy()


def memory_footprint_bytes(n_vectors: int, d: int, bit_width: int) -> dict:
    """Byte breakdown of a TurboQuant-compressed cache (turboquant/utils.py:101-123):
    (b-1)-bit indices, 1-bit signs, one float32 norm per vector."""
    mse_bytes = -(-n_vectors * d * (bit_width - 1) // 8)
    qjl_bytes = -(-n_vectors * d // 8)
    norm_bytes = 4 * n_vectors
    total = mse_bytes + qjl_bytes + norm_bytes
    original = 2 * n_vectors * d
    return {
        "mse_indices_bytes": int(mse_bytes),
        "qjl_signs_bytes": int(qjl_bytes),
        "norms_bytes": norm_bytes,
        "total_bytes": int(total),
        "original_fp16_bytes": original,
        "compression_ratio": original / total if total > 0 else float("inf"),
    }
