"""Rotation primitives with the reference's names and signatures
(turboquant/rotation.py:25-185).

Table generation (seeded NumPy draws, QR) stays on the host because parity
with the reference's random streams requires NumPy's generators; applying a
rotation to vectors runs on the GPU through the C ABI (tq_fwht / tq_rotate).
"""
from __future__ import annotations

import ctypes as C
from collections import OrderedDict

import numpy as np

from . import _lib as L


def random_rotation_dense(d: int, rng: np.random.Generator) -> np.ndarray:
    """Haar-distributed rotation, det +1 (turboquant/rotation.py:25-50)."""
    if d < 1:
        raise ValueError(f"d must be >= 1, got {d}")
    q, r = np.linalg.qr(rng.standard_normal((d, d)))
    flip = np.sign(np.diag(r))
    flip[flip == 0] = 1.0
    q = q * flip[None, :]
    if np.linalg.slogdet(q)[0] < 0:
        q[:, 0] = -q[:, 0]
    return q


def _next_power_of_2(n: int) -> int:
    p = 1
    while p < n:
        p <<= 1
    return p


def hadamard_matrix(n: int) -> np.ndarray:
    """Unnormalised +-1 Sylvester-Hadamard matrix (turboquant/rotation.py:61-72):
    entry (i, j) = (-1)^popcount(i & j)."""
    if n < 1 or n & (n - 1):
        raise ValueError(f"n must be a positive power of 2, got {n}")
    i = np.arange(n)
    parity = np.zeros((n, n), dtype=np.int64)
    both = i[:, None] & i[None, :]
    while both.any():
        parity ^= both & 1
        both >>= 1
    return 1.0 - 2.0 * parity


def random_rotation_fast(d: int, rng: np.random.Generator):
    """(signs1, signs2, padded_d): two `choice` draws in that order
    (turboquant/rotation.py:75-96)."""
    padded_d = _next_power_of_2(d)
    signs1 = rng.choice([-1.0, 1.0], size=padded_d)
    signs2 = rng.choice([-1.0, 1.0], size=padded_d)
    return signs1, signs2, padded_d


def fast_walsh_hadamard_transform(x: np.ndarray) -> np.ndarray:
    """Normalised WHT of one vector, float64 on the GPU with the reference's
    butterfly order (turboquant/rotation.py:99-121)."""
    x = np.asarray(x)
    n = len(x)
    if n < 1 or n & (n - 1):
        raise ValueError(f"Input length must be a positive power of 2, got {n}")
    tt = L.torch()
    xd = L.to_device(x.astype(np.float64))
    yd = tt.empty_like(xd)
    L.check(L.lib().tq_fwht(L.ptr(xd), L.ptr(yd), 1, n, L.TQ_F64, L.TQ_F64, L.stream_ptr()))
    return yd.cpu().numpy()


_sign_handles: "OrderedDict[tuple, L.Handle]" = OrderedDict()


def _sign_handle(d, signs1, signs2, padded_d) -> L.Handle:
    s1 = np.ascontiguousarray(signs1, dtype=np.float64)
    s2 = np.ascontiguousarray(signs2, dtype=np.float64)
    if len(s1) != padded_d or len(s2) != padded_d or padded_d != _next_power_of_2(d):
        raise ValueError(f"sign vectors must have length padded_d={padded_d} = next power of 2 of d={d}")
    key = (d, s1.tobytes(), s2.tobytes())
    h = _sign_handles.get(key)
    if h is None:
        h = L.Handle(d, 1, np.array([-1.0, 1.0]), signs1=s1, signs2=s2)
        _sign_handles[key] = h
        while len(_sign_handles) > 16:
            _sign_handles.popitem(last=False)
    else:
        _sign_handles.move_to_end(key)
    return h


def _apply(x2d, signs1, signs2, padded_d, transpose):
    tt = L.torch()
    n, d = x2d.shape
    h = _sign_handle(d, signs1, signs2, padded_d)
    xd = L.to_device(np.asarray(x2d, dtype=np.float64))
    yd = tt.empty_like(xd)
    L.check(L.lib().tq_rotate(h.h, L.ptr(xd), L.ptr(yd), n, L.TQ_F64, L.TQ_F64, int(transpose), L.stream_ptr()))
    return yd.cpu().numpy()


def apply_fast_rotation(x, signs1, signs2, padded_d):
    """D2 H D1 x for one vector (turboquant/rotation.py:124-145)."""
    return _apply(np.asarray(x)[None, :], signs1, signs2, padded_d, False)[0]


def apply_fast_rotation_transpose(y, signs1, signs2, padded_d):
    """D1 H D2 y for one vector (turboquant/rotation.py:148-160)."""
    return _apply(np.asarray(y)[None, :], signs1, signs2, padded_d, True)[0]


def apply_fast_rotation_batch(X, signs1, signs2, padded_d):
    """D2 H D1 on every row of X (turboquant/rotation.py:163-185)."""
    return _apply(np.asarray(X), signs1, signs2, padded_d, False)
