"""CPU oracle for the TurboQuant+ KV-codec / compressed-KV attention path.

TEST INFRASTRUCTURE ONLY.  This module is the checker: tests, the smoke check
and the CPU-baseline leg of the benchmark may import it.  The shipped package
never does; its per-vector work runs in HIP kernels and fails loudly when the
HIP library is missing.

Everything here is float64 NumPy written to follow the reference's arithmetic
step by step (citations are file:line in the reference tree):

  rotation      turboquant/rotation.py:25-185
  codebook      turboquant/codebook.py:29-134
  PolarQuant    turboquant/polar_quant.py:46-132
  QJL           turboquant/qjl.py:32-134
  TurboQuant    turboquant/turboquant.py:33-171
  KV cache      turboquant/kv_cache.py:30-188
  bit packing   turboquant/utils.py:20-123
  outlier split turboquant/outlier.py:45-217
  temporal decay benchmarks/temporal_decay_prototype.py:93-125

Pinned by (see tests/test_oracle_*.py): golden vectors written from the
reference itself (tests/golden/), scipy.linalg.hadamard, brute-force argmin,
closed-form centroids and conditional expectations, orthogonality, literal
pack bytes and size arithmetic.

Functions the reference holds no code for, and what pins them instead
(tests/test_oracle_math.py):
  `q8_0_quantize`/`q8_0_dequantize`  ggml's published quantize_row_q8_0 (d = amax/127
      kept in fp32, id = 1/d, roundf(x*id), d stored as fp16), on literal blocks: ties at
      +-0.5/1.5/2.5, the largest float below one half, a zero block, a scale that changes
      when rounded to fp16;
  `decode_attention`, Sparse-V branch  hand-built cases whose skipped set and output are
      written down (running maximum vs the split's final one, a maximum not carried
      across splits, weight == tau kept, split bounds for a ragged tile count);
  `score_tile`, `gaussian` projection  regression slope of the reconstruction on the true
      residual (1 only for the scale sqrt(pi/2)/d);
  `fork_blocks_pack`/`fork_blocks_unpack`  the extraction formulas the reference's documents
      print, applied element by element.  No block written by the fork itself is available:
      parity with the fork's bytes stays unpinned.
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field

import numpy as np
from scipy import stats

SQRT_HALF_PI = math.sqrt(math.pi / 2.0)  # qjl.py:32


# --------------------------------------------------------------------------
# rotation primitives (rotation.py)
# --------------------------------------------------------------------------

def haar_rotation(d: int, rng: np.random.Generator) -> np.ndarray:
    """Haar rotation with det +1 (rotation.py:25-50)."""
    if d < 1:
        raise ValueError(f"d must be >= 1, got {d}")
    g = rng.standard_normal((d, d))
    q, r = np.linalg.qr(g)
    s = np.sign(np.diag(r))
    s[s == 0] = 1.0
    q = q * s[None, :]
    if np.linalg.slogdet(q)[0] < 0:
        q[:, 0] = -q[:, 0]
    return q


def next_pow2(n: int) -> int:
    """rotation.py:53-58."""
    p = 1
    while p < n:
        p <<= 1
    return p


def sylvester_hadamard(n: int) -> np.ndarray:
    """Unnormalised +-1 Sylvester matrix (rotation.py:61-72)."""
    if n < 1 or n & (n - 1):
        raise ValueError(f"n must be a positive power of 2, got {n}")
    h = np.ones((1, 1))
    while h.shape[0] < n:
        h = np.block([[h, h], [h, -h]])
    return h


def sign_diagonals(d: int, rng: np.random.Generator):
    """(signs1, signs2, padded_d); two `choice` draws in this order (rotation.py:75-96)."""
    pd = next_pow2(d)
    s1 = rng.choice([-1.0, 1.0], size=pd)
    s2 = rng.choice([-1.0, 1.0], size=pd)
    return s1, s2, pd


def fwht(x: np.ndarray) -> np.ndarray:
    """Normalised natural-order WHT over the last axis (rotation.py:99-121).

    Stage order h = 1, 2, 4, ...; pair (j, j+h) -> (a+b, a-b); one division by
    sqrt(n) at the end.  Vectorised over leading axes, same additions per row.
    """
    x = np.array(x, dtype=np.float64)
    n = x.shape[-1]
    if n < 1 or n & (n - 1):
        raise ValueError(f"Input length must be a positive power of 2, got {n}")
    lead = x.shape[:-1]
    h = 1
    while h < n:
        v = x.reshape(lead + (n // (2 * h), 2, h))
        a = v[..., 0, :].copy()
        b = v[..., 1, :].copy()
        v[..., 0, :] = a + b
        v[..., 1, :] = a - b
        x = v.reshape(lead + (n,))
        h *= 2
    return x / np.sqrt(n)


def rotate_fast(x, s1, s2, pd, transpose=False):
    """D2 H D1 x (or its transpose D1 H D2 y) on the last axis, with zero
    padding to `pd` and truncation back (rotation.py:124-185)."""
    x = np.asarray(x, dtype=np.float64)
    d = x.shape[-1]
    buf = np.zeros(x.shape[:-1] + (pd,))
    buf[..., :d] = x
    first, second = (s2, s1) if transpose else (s1, s2)
    buf = buf * first
    buf = fwht(buf)
    buf = buf * second
    return buf[..., :d]


# --------------------------------------------------------------------------
# codebook (codebook.py)
# --------------------------------------------------------------------------

def gauss_cond_mean(sigma: float, a: float, b: float) -> float:
    """E[X | a < X < b], X ~ N(0, sigma^2), with the reference's tail
    fallbacks when the interval mass is below 1e-15 (codebook.py:88-118)."""
    za = a / sigma if np.isfinite(a) else a
    zb = b / sigma if np.isfinite(b) else b
    if not np.isfinite(za):
        mass = stats.norm.cdf(zb)
    elif not np.isfinite(zb):
        mass = stats.norm.sf(za)
    else:
        mass = stats.norm.cdf(zb) - stats.norm.cdf(za)
    if mass < 1e-15:
        if np.isfinite(a) and not np.isfinite(b):
            return a + sigma
        if not np.isfinite(a) and np.isfinite(b):
            return b - sigma
        if np.isfinite(a) and np.isfinite(b):
            return (a + b) / 2.0
        return 0.0
    return sigma * (stats.norm.pdf(za) - stats.norm.pdf(zb)) / mass


def lloyd_gaussian(n_levels: int, sigma: float, n_iter: int = 100) -> np.ndarray:
    """Quantile-initialised Lloyd iteration, exactly `n_iter` rounds after the
    initial centroid pass (codebook.py:52-85)."""
    edges = stats.norm.ppf(np.linspace(0, 1, n_levels + 1)[1:-1], scale=sigma)
    c = np.zeros(n_levels)

    def refresh(edges):
        c[0] = gauss_cond_mean(sigma, -np.inf, edges[0])
        for i in range(1, n_levels - 1):
            c[i] = gauss_cond_mean(sigma, edges[i - 1], edges[i])
        c[-1] = gauss_cond_mean(sigma, edges[-1], np.inf)

    refresh(edges)
    for _ in range(n_iter):
        edges = (c[:-1] + c[1:]) / 2.0
        refresh(edges)
    return np.sort(c)


def centroids_for(bits: int, d: int) -> np.ndarray:
    """codebook.py:29-49."""
    if bits == 1:
        c = np.sqrt(2.0 / (np.pi * d))
        return np.array([-c, c])
    if bits == 2:
        return np.array([-1.51, -0.453, 0.453, 1.51]) / np.sqrt(d)
    return lloyd_gaussian(1 << bits, sigma=1.0 / np.sqrt(d))


def midpoints(centroids: np.ndarray) -> np.ndarray:
    return (centroids[:-1] + centroids[1:]) / 2.0


def nearest_index(values: np.ndarray, centroids: np.ndarray) -> np.ndarray:
    """Index = number of midpoints strictly below the value; a value equal to
    a midpoint takes the lower index (codebook.py:121-134)."""
    values = np.asarray(values)
    return np.searchsorted(midpoints(centroids), values.ravel()).reshape(values.shape)


# --------------------------------------------------------------------------
# quantisers (polar_quant.py, qjl.py, turboquant.py, kv_cache.py)
# --------------------------------------------------------------------------

class PolarRef:
    """polar_quant.py:46-132.  `rotation="dense"` is the class as written;
    `rotation="wht"` swaps in D2 H D1 with signs drawn as rotation.py:94-95
    from the same seeded generator (signs2 forced to ones when
    `single_diagonal`)."""

    def __init__(self, d, bit_width, seed=42, norm_correction=True,
                 rotation="dense", single_diagonal=False):
        self.d, self.bit_width = d, bit_width
        self.n_centroids = 1 << bit_width
        self.norm_correction = norm_correction
        self.mode = rotation
        rng = np.random.default_rng(seed)
        if rotation == "dense":
            self.rotation = haar_rotation(d, rng)
        else:
            self.s1, self.s2, self.pd = sign_diagonals(d, rng)
            if single_diagonal:
                self.s2 = np.ones_like(self.s2)
        self.centroids = centroids_for(bit_width, d)

    def _fwd(self, x):
        if self.mode == "dense":
            return (self.rotation @ x.T).T
        return rotate_fast(x, self.s1, self.s2, self.pd)

    def _inv(self, y):
        if self.mode == "dense":
            return (self.rotation.T @ y.T).T
        return rotate_fast(y, self.s1, self.s2, self.pd, transpose=True)

    def rotated(self, x):
        """Rotated unit vectors (the values the index decision is made on)."""
        x = np.atleast_2d(np.asarray(x, dtype=np.float64))
        n = np.linalg.norm(x, axis=1)
        safe = np.where(n > 0, n, 1.0)
        return self._fwd(x / safe[:, None]), n

    def quantize(self, x):
        x = np.asarray(x)
        single = x.ndim == 1
        y, n = self.rotated(x)
        idx = nearest_index(y, self.centroids)
        return (idx[0], n[0]) if single else (idx, n)

    def dequantize(self, indices, norms):
        indices = np.asarray(indices)
        single = indices.ndim == 1
        if single:
            indices = indices[None, :]
            norms = np.array([norms])
        y = self.centroids[indices]
        if self.norm_correction:
            yn = np.linalg.norm(y, axis=1, keepdims=True)
            yn = np.where(yn > 1e-10, yn, 1.0)
            y = y / yn
        out = self._inv(y) * np.asarray(norms)[:, None]
        return out[0] if single else out

    def quantize_and_residual(self, x):
        idx, n = self.quantize(x)
        return idx, n, x - self.dequantize(idx, n)


class QJLRef:
    """qjl.py:50-134.  `projection="orthogonal"` is the class as written (QR of
    the Gaussian, scale sqrt(pi/2)/sqrt(d)); `projection="gaussian"` keeps the
    raw Gaussian matrix with scale sqrt(pi/2)/d (PLAN.md:71-77)."""

    def __init__(self, d, seed=123, projection="orthogonal"):
        self.d = d
        g = np.random.default_rng(seed).standard_normal((d, d))
        if projection == "orthogonal":
            q, r = np.linalg.qr(g)
            self.S = q * np.sign(np.diag(r))[None, :]
            self.scale = SQRT_HALF_PI / np.sqrt(d)
        else:
            self.S = g
            self.scale = SQRT_HALF_PI / d

    def quantize(self, r):
        r = np.asarray(r)
        single = r.ndim == 1
        if single:
            r = r[None, :]
        n = np.linalg.norm(r, axis=1)
        z = np.sign((self.S @ r.T).T).astype(np.int8)
        z[z == 0] = 1
        return (z[0], n[0]) if single else (z, n)

    def project(self, r):
        """S r (the values the sign decision is made on)."""
        r = np.atleast_2d(np.asarray(r, dtype=np.float64))
        return (self.S @ r.T).T

    def dequantize(self, signs, norms, shrinkage=1.0):
        signs = np.asarray(signs)
        single = signs.ndim == 1
        if single:
            signs = signs[None, :]
            norms = np.array([norms])
        out = (self.S.T @ signs.astype(np.float64).T).T
        out = out * ((self.scale * np.asarray(norms))[:, None] * shrinkage)
        return out[0] if single else out


@dataclass
class CompressedRef:
    mse_indices: np.ndarray
    vector_norms: np.ndarray
    qjl_signs: np.ndarray
    residual_norms: np.ndarray
    bit_width: int


class TurboRef:
    """turboquant.py:43-149: PolarQuant(b-1, seed) + QJL(seed+1000)."""

    def __init__(self, d, bit_width, seed=42, norm_correction=True,
                 rotation="dense", projection="orthogonal"):
        if bit_width < 2:
            raise ValueError("TurboQuant requires bit_width >= 2")
        self.d, self.bit_width = d, bit_width
        self.polar_quant = PolarRef(d, bit_width - 1, seed, norm_correction, rotation)
        self.qjl = QJLRef(d, seed + 1000, projection)

    def quantize(self, x):
        idx, n, res = self.polar_quant.quantize_and_residual(x)
        z, rn = self.qjl.quantize(res)
        return CompressedRef(idx, n, z, rn, self.bit_width)

    def dequantize(self, c, shrinkage=1.0):
        return (self.polar_quant.dequantize(c.mse_indices, c.vector_norms)
                + self.qjl.dequantize(c.qjl_signs, c.residual_norms, shrinkage))

    def compressed_size_bits(self, n_vectors):
        return n_vectors * (self.d * self.bit_width + 32)

    def compression_ratio(self, original_bits_per_value=16):
        return self.d * original_bits_per_value / (self.d * self.bit_width + 32)


class TurboMSERef:
    """turboquant.py:152-171."""

    def __init__(self, d, bit_width, seed=42, norm_correction=True, rotation="dense"):
        self.d, self.bit_width = d, bit_width
        self.polar_quant = PolarRef(d, bit_width, seed, norm_correction, rotation)

    def quantize(self, x):
        return self.polar_quant.quantize(x)

    def dequantize(self, idx, norms):
        return self.polar_quant.dequantize(idx, norms)


def channel_split(d: int, target_bits: float):
    """outlier.py:45-67: (n_outlier, high_bits, n_normal, low_bits); the high-rate
    channels are the first round(d * frac) ones."""
    low = int(np.floor(target_bits))
    n_out = int(round(d * (target_bits - low)))
    return n_out, low + 1, d - n_out, low


class OutlierRef:
    """outlier.py:70-217: channels 0..n_outlier-1 through PolarQuant(high-1 bits, seed),
    the rest through PolarQuant(low-1 bits, seed+500), QJL(seed+1000) on the full residual.
    Returns plain tuples (outlier idx, outlier norms, normal idx, normal norms, signs,
    residual norms)."""

    def __init__(self, d, target_bits, seed=42):
        self.d, self.target_bits = d, target_bits
        self.n_outlier, self.high_bits, self.n_normal, self.low_bits = channel_split(d, target_bits)
        self.effective_bits = (self.n_outlier * self.high_bits + self.n_normal * self.low_bits) / d
        self.pq_outlier = PolarRef(self.n_outlier, self.high_bits - 1, seed) if self.n_outlier > 0 else None
        self.pq_normal = PolarRef(self.n_normal, self.low_bits - 1, seed + 500) if self.n_normal > 0 else None
        self.qjl = QJLRef(d, seed + 1000)

    def quantize(self, x):
        x = np.asarray(x, dtype=np.float64)
        single = x.ndim == 1
        xb = x[None] if single else x
        parts, res = [], np.zeros_like(xb)
        for pq, sl in ((self.pq_outlier, slice(0, self.n_outlier)), (self.pq_normal, slice(self.n_outlier, self.d))):
            if pq is None:
                parts += [np.array([]), np.array([])]
                continue
            sub = xb[:, np.arange(sl.start, sl.stop)]    # gathered as the reference does (outlier.py:119-120): the
                                                         # memory order of the result decides the summation order of the norm
            idx, n, r = pq.quantize_and_residual(sub if xb.shape[0] > 1 else sub[0])   # outlier.py:124,132
            res[:, sl] = r
            parts += [idx, n]
        z, rn = self.qjl.quantize(res[0] if single else res)
        return (*parts, z, rn)

    def dequantize(self, c):
        oi, on, ni, nn, z, rn = c
        xq = self.qjl.dequantize(z, rn)
        out = np.zeros_like(xq)
        if self.pq_outlier is not None:
            out[..., :self.n_outlier] = self.pq_outlier.dequantize(oi, on)
        if self.pq_normal is not None:
            out[..., self.n_outlier:] = self.pq_normal.dequantize(ni, nn)
        return out + xq

    def compression_ratio(self, original_bits=16):
        return self.d * original_bits / (self.d * self.effective_bits + 32 + 64)   # outlier.py:209-217


@dataclass
class CompressedKVRef:
    k_compressed: list = field(default_factory=list)
    v_indices: list = field(default_factory=list)
    v_norms: list = field(default_factory=list)
    num_layers: int = 0
    num_heads: int = 0
    seq_len: int = 0
    head_dim: int = 0
    k_bit_width: int = 0
    v_bit_width: int = 0


class KVRef:
    """kv_cache.py:69-188: K through TurboRef(seed), V through
    TurboMSERef(seed+500); one quantiser each, shared by all layers/heads."""

    def __init__(self, head_dim, k_bits=3, v_bits=3, seed=42, norm_correction=True):
        self.head_dim, self.k_bits, self.v_bits = head_dim, k_bits, v_bits
        self.k_quantizer = TurboRef(head_dim, k_bits, seed, norm_correction)
        self.v_quantizer = TurboMSERef(head_dim, v_bits, seed + 500, norm_correction)

    def compress(self, k, v):
        L, H, S, D = k.shape
        assert D == self.head_dim
        assert v.shape == k.shape
        out = CompressedKVRef(num_layers=L, num_heads=H, seq_len=S, head_dim=D,
                              k_bit_width=self.k_bits, v_bit_width=self.v_bits)
        for l in range(L):
            kc, vi, vn = [], [], []
            for h in range(H):
                kc.append(self.k_quantizer.quantize(k[l, h]))
                i, n = self.v_quantizer.quantize(v[l, h])
                vi.append(i)
                vn.append(n)
            out.k_compressed.append(kc)
            out.v_indices.append(vi)
            out.v_norms.append(vn)
        return out

    def decompress(self, c):
        k = np.zeros((c.num_layers, c.num_heads, c.seq_len, c.head_dim))
        v = np.zeros_like(k)
        for l in range(c.num_layers):
            for h in range(c.num_heads):
                k[l, h] = self.k_quantizer.dequantize(c.k_compressed[l][h])
                v[l, h] = self.v_quantizer.dequantize(c.v_indices[l][h], c.v_norms[l][h])
        return k, v

    def memory_stats(self, seq_len, num_layers, num_heads):
        n = num_layers * num_heads * seq_len
        orig = n * self.head_dim * 2
        comp = (n * (self.head_dim * self.k_bits + 32) + n * self.head_dim * self.v_bits) / 8
        return {"original_mb": orig / 1024 / 1024, "compressed_mb": comp / 1024 / 1024,
                "compression_ratio": orig / comp,
                "k_bits_per_value": self.k_bits, "v_bits_per_value": self.v_bits}


# --------------------------------------------------------------------------
# host bit packing (utils.py)
# --------------------------------------------------------------------------

def pack_sign_bits(signs: np.ndarray) -> np.ndarray:
    """+1 -> bit 1, first element in the MSB, zero padded to a byte (utils.py:20-49)."""
    bits = (np.asarray(signs) > 0).astype(np.uint8)
    return np.packbits(bits, axis=-1)


def unpack_sign_bits(packed: np.ndarray, d: int) -> np.ndarray:
    """utils.py:52-68."""
    bits = np.unpackbits(np.asarray(packed, dtype=np.uint8), axis=-1)[..., :d]
    return bits.astype(np.int8) * 2 - 1


def pack_index_stream(indices: np.ndarray, bit_width: int) -> np.ndarray:
    """One MSB-first bit stream over the flattened array for b <= 4, one byte
    per index above (utils.py:71-98)."""
    if bit_width <= 0 or bit_width > 8:
        raise ValueError(f"bit_width must be 1-8, got {bit_width}")
    if bit_width > 4:
        return np.asarray(indices).astype(np.uint8)
    flat = np.asarray(indices).ravel().astype(np.uint8)
    shifts = np.arange(bit_width - 1, -1, -1, dtype=np.uint8)
    bits = (flat[:, None] >> shifts[None, :]) & 1
    return np.packbits(bits.ravel())


def footprint(n_vectors: int, d: int, bit_width: int) -> dict:
    """utils.py:101-123."""
    mse = int(np.ceil(n_vectors * d * (bit_width - 1) / 8))
    qjl = int(np.ceil(n_vectors * d / 8))
    norms = n_vectors * 4
    total = mse + qjl + norms
    orig = n_vectors * d * 2
    return {"mse_indices_bytes": mse, "qjl_signs_bytes": qjl, "norms_bytes": norms,
            "total_bytes": total, "original_fp16_bytes": orig,
            "compression_ratio": orig / total if total > 0 else float("inf")}


# --------------------------------------------------------------------------
# production ("turboN") format: WHT rotation, write-side corrected fp16 norm
# --------------------------------------------------------------------------
# Arithmetic follows benchmarks/temporal_decay_prototype.py:58-90 (midpoint
# digitise, corrected norm = norm / ||centroids[idx]|| with the > 1e-10 guard)
# composed with rotation.py:163-185; the only addition is rounding the stored
# norm to fp16, which the device format requires.

def turbo_encode(x, s1, s2, centroids, norm_dtype=np.float16, norm_correction=True):
    """-> (idx uint8 [n,d], stored norm [n] in `norm_dtype`, y fp64 [n,d]).

    y is the rotated unit vector the index decision was made on (used for the
    decision-boundary band accounting).  A zero vector stores norm 0.
    """
    x = np.atleast_2d(np.asarray(x, dtype=np.float64))
    d = x.shape[1]
    n = np.linalg.norm(x, axis=1)
    safe = np.where(n > 0, n, 1.0)
    y = rotate_fast(x / safe[:, None], s1, s2, len(s1))
    idx = nearest_index(y, centroids)
    if norm_correction:
        cn = np.linalg.norm(centroids[idx], axis=1)
        g = n / np.where(cn > 1e-10, cn, 1.0)
    else:
        g = n
    return idx.astype(np.uint8), g.astype(norm_dtype), y


def turbo_decode_rotated(idx, g, centroids):
    """Rotated-domain reconstruction g * centroids[idx] (fp64)."""
    return centroids[np.asarray(idx, dtype=np.int64)] * np.asarray(g, dtype=np.float64)[..., None]


def turbo_decode(idx, g, centroids, s1, s2):
    """Original-domain reconstruction R^T (g * centroids[idx])."""
    return rotate_fast(turbo_decode_rotated(idx, g, centroids), s1, s2, len(s1), transpose=True)


def requantize(idx_src, g_src, cent_src, cent_dst, mid_dst=None):
    """Temporal decay of a stored row to a narrower codebook, in the rotated domain
    (benchmarks/temporal_decay_prototype.py:93-125, `requantize_3to2`): decode with the
    stored (corrected) norm, renormalise, nearest narrower centroid by np.digitize over
    the midpoints (a value equal to a midpoint takes the HIGHER index, unlike
    nearest_index), corrected norm for the new codes.  Rows are independent."""
    idx_src = np.asarray(idx_src)
    g_src = np.asarray(g_src, dtype=np.float64)
    mid = midpoints(cent_dst) if mid_dst is None else np.asarray(mid_dst, dtype=np.float64)
    idx_out = np.zeros(idx_src.shape, dtype=np.uint8)
    g_out = np.zeros(g_src.shape, dtype=np.float64)
    for r in range(idx_src.shape[0]):
        values = cent_src[idx_src[r]] * g_src[r]
        recon = np.linalg.norm(values)
        if recon > 1e-10:
            normalized = values / recon
        else:
            normalized, recon = values, 0.0
        i2 = np.digitize(normalized, mid)
        cn = np.sqrt(np.sum(cent_dst[i2] ** 2))
        idx_out[r] = i2
        g_out[r] = recon / cn if cn > 1e-10 else recon
    return idx_out, g_out


def boundary_band_mismatches(y, idx_test, centroids, rel=1e-6):
    """Classify index mismatches against the fp64 decision values `y`.

    A mismatch is admissible iff y lies within rel * max(|b|, 1/sqrt(d)) of
    every decision boundary b between the oracle index and the tested index.
    Returns (n_mismatch, n_inadmissible).
    """
    y = np.asarray(y, dtype=np.float64)
    d = y.shape[-1]
    b = midpoints(centroids)
    ref = np.searchsorted(b, y.ravel()).reshape(y.shape)
    test = np.asarray(idx_test).astype(np.int64)
    bad = ref != test
    n_bad = int(bad.sum())
    if n_bad == 0:
        return 0, 0
    yb, rb, tb = y[bad], ref[bad], test[bad]
    lo, hi = np.minimum(rb, tb), np.maximum(rb, tb)
    inadmissible = 0
    for v, l, h in zip(yb, lo, hi):
        crossed = b[l:h]
        tol = rel * np.maximum(np.abs(crossed), 1.0 / np.sqrt(d))
        if not np.all(np.abs(v - crossed) <= tol):
            inadmissible += 1
    return n_bad, inadmissible


# ---- device layout: "pair containers" in 128-token blocks ------------------
# A ROW holds 64 pair codes (128 values) in 16*b bytes; pair p = (lo | hi << b).
# A row is four groups of 16 pairs (group g = pairs 16g..16g+15); a group owns b
# dwords, and dword j of group g is row dword 4j + g, i.e. 16-byte chunk j of the row
# holds dword j of the four groups.  Inside a group, pair k sits in
#   b = 4 : byte k%4 of dword k//4
#   b = 2 : nibble k%8 of dword k//8
#   b = 3 : bits 6*(k%4).. of dword k//4 for k < 12; pairs 12..15 are a 24-bit tail (pair k at tail
#           bit 6*(k-12)), byte j of which is the top byte of dword j.
# Pairs 2q, 2q+1 ("quad" q: four values) are contiguous bits in every width, so a reader can index
# a table by a whole quad.
# K rows: row = token, pair p = dims (2p, 2p+1).
# V rows are dim-major inside each 64-token tile: row (token & 64) | (dim & 63)
#         holds dims r and 64+r of the tile's 64 tokens; tokens 2*tp and 2*tp+1 of
#         the tile (lo, hi) of dim half hf = dim >> 6 are pair 4*(tp//2) + 2*hf + tp%2: a quad is four
#         consecutive tokens of one dim.
# A BLOCK is 128 rows stored chunk-major: [16*b/16 chunks][128 rows][16 B],
# followed by 128 fp16 norms (token order).  Block bytes = 128*(16*b + 2).

ROWS_PER_BLOCK = 128


def row_bytes(bits: int) -> int:
    return 16 * bits


def block_bytes(bits: int) -> int:
    return ROWS_PER_BLOCK * (row_bytes(bits) + 2)


def _pairs_to_rows(pairs: np.ndarray, bits: int) -> np.ndarray:
    """pairs [..., 64] (values < 4**bits) -> row dwords [..., 4*bits] uint32.

    A row is four groups of 16 pairs; group g owns `bits` dwords, and dword j
    of group g is row dword 4*j + g (so 16-byte chunk j of the row holds dword
    j of the four groups).  Inside a group: 4-bit pair k = byte k%4 of dword
    k/4; 2-bit pair k = nibble k%8 of dword k/8; 3-bit pair k < 12 = bits
    6*(k%4).. of dword k/4, and pairs 12..15 form a 24-bit tail (pair k at tail
    bit 6*(k-12)) whose byte j is the top byte of dword j.  Two adjacent pairs
    2q, 2q+1 (a "quad" of four values) are contiguous bits in every width."""
    pairs = pairs.astype(np.uint32)
    lead = pairs.shape[:-1]
    grp = pairs.reshape(lead + (4, 16))
    out = np.zeros(lead + (4 * bits,), dtype=np.uint32)
    if bits not in (2, 3, 4):
        raise ValueError("bits must be 2, 3 or 4")
    per, width = {4: (4, 8), 2: (8, 4), 3: (4, 6)}[bits]
    for g in range(4):
        for k in range(16 if bits != 3 else 12):
            out[..., 4 * (k // per) + g] |= grp[..., g, k] << np.uint32(width * (k % per))
        if bits == 3:
            tail = np.zeros(lead, dtype=np.uint32)
            for k in range(12, 16):
                tail |= grp[..., g, k] << np.uint32(6 * (k - 12))
            for j in range(3):
                out[..., 4 * j + g] |= ((tail >> np.uint32(8 * j)) & np.uint32(0xFF)) << np.uint32(24)
    return out


def _rows_to_pairs(rows: np.ndarray, bits: int) -> np.ndarray:
    rows = rows.astype(np.uint32)
    if bits not in (2, 3, 4):
        raise ValueError("bits must be 2, 3 or 4")
    per, width = {4: (4, 8), 2: (8, 4), 3: (4, 6)}[bits]
    mask = np.uint32((1 << width) - 1)
    cols = []
    for g in range(4):
        for k in range(16 if bits != 3 else 12):
            cols.append((rows[..., 4 * (k // per) + g] >> np.uint32(width * (k % per))) & mask)
        if bits == 3:
            tail = ((rows[..., g] >> np.uint32(24)) | ((rows[..., 4 + g] >> np.uint32(24)) << np.uint32(8))
                    | ((rows[..., 8 + g] >> np.uint32(24)) << np.uint32(16)))
            for k in range(12, 16):
                cols.append((tail >> np.uint32(6 * (k - 12))) & mask)
    return np.stack(cols, axis=-1)


def layout_pack(idx: np.ndarray, g: np.ndarray, bits: int, kind: str) -> np.ndarray:
    """idx [T,128] (T multiple of 128), g [T] fp16 -> uint8 [T/128 * block_bytes]."""
    idx = np.asarray(idx).astype(np.uint32)
    T, d = idx.shape
    assert d == 128 and T % ROWS_PER_BLOCK == 0
    nb = T // ROWS_PER_BLOCK
    if kind == "k":
        pairs = idx[:, 0::2] | (idx[:, 1::2] << np.uint32(bits))          # [T,64]
    else:
        q = idx.reshape(T // 64, 16, 2, 2, 2, 64)                          # tile, token quad, pair in quad, parity, dim half, r
        lo = q[:, :, :, 0].transpose(0, 4, 1, 3, 2)                        # tile, r, token quad, dim half, pair in quad
        hi = q[:, :, :, 1].transpose(0, 4, 1, 3, 2)
        pairs = (lo | (hi << np.uint32(bits))).reshape(T, 64)              # row = 64*tile + r; pair = 4*tq + 2*half + tp%2
    rows = _pairs_to_rows(pairs, bits)                                     # [T, 4*bits]
    rows = rows.reshape(nb, ROWS_PER_BLOCK, bits, 4).transpose(0, 2, 1, 3) # block, chunk, row, 4
    out = np.zeros((nb, block_bytes(bits)), dtype=np.uint8)
    code_bytes = ROWS_PER_BLOCK * row_bytes(bits)
    out[:, :code_bytes] = np.ascontiguousarray(rows).astype("<u4").view(np.uint8).reshape(nb, code_bytes)
    out[:, code_bytes:] = np.asarray(g, dtype=np.float16).reshape(nb, ROWS_PER_BLOCK).view(np.uint8)
    return out.reshape(-1)


def layout_unpack(buf: np.ndarray, bits: int, kind: str):
    """Inverse of layout_pack -> (idx uint8 [T,128], g fp16 [T])."""
    bb = block_bytes(bits)
    buf = np.asarray(buf, dtype=np.uint8).reshape(-1, bb)
    nb = buf.shape[0]
    T = nb * ROWS_PER_BLOCK
    code_bytes = ROWS_PER_BLOCK * row_bytes(bits)
    rows = np.ascontiguousarray(buf[:, :code_bytes]).view("<u4").reshape(nb, bits, ROWS_PER_BLOCK, 4)
    rows = rows.transpose(0, 2, 1, 3).reshape(T, 4 * bits)
    g = np.ascontiguousarray(buf[:, code_bytes:]).view(np.float16).reshape(T)
    pairs = _rows_to_pairs(rows, bits)
    mask = np.uint32((1 << bits) - 1)
    lo, hi = pairs & mask, (pairs >> np.uint32(bits)) & mask
    idx = np.zeros((T, 128), dtype=np.uint8)
    if kind == "k":
        idx[:, 0::2] = lo
        idx[:, 1::2] = hi
    else:
        q = np.zeros((T // 64, 16, 2, 2, 2, 64), dtype=np.uint8)           # tile, token quad, pair in quad, parity, dim half, r
        q[:, :, :, 0] = lo.reshape(T // 64, 64, 16, 2, 2).transpose(0, 2, 4, 3, 1)
        q[:, :, :, 1] = hi.reshape(T // 64, 64, 16, 2, 2).transpose(0, 2, 4, 3, 1)
        idx = q.reshape(T, 128)
    return idx, g


# --------------------------------------------------------------------------
# Per-128 block layout of the llama.cpp fork, as its documents state it (no code for it exists in
# the reference tree, so parity with the fork itself is unpinned): one block per 128-value vector,
#   turbo3: norm fp16 | qs[32] | signs[16]  (50 B), idx = low2 | hi1 << 2,
#           low2 = (qs[j/4] >> ((j%4)*2)) & 3, hi1 = (signs[j/8] >> (j%8)) & 1
#           (docs/papers/block-size-experiment.md:33-39, docs/papers/turbo4-resurrection.md:130-134)
#   turbo4: norm fp16 | rnorm fp16 | qs[64]  (68 B = 4.25 bits per value: turbo4-resurrection.md:208 "qs[64],
#           maintaining the 68-byte block size", README.md:43,94), idx = (qs[j/2] >> ((j%2)*4)) & 0xF
#           (turbo4-resurrection.md:169).  rnorm is the residual-norm field the struct keeps from the 3-bit + QJL
#           turbo4 (docs/turbo4-investigation.md:42-49); 4-bit PolarQuant does not use it: packed as 0, ignored
#           when unpacked.  Its position (right after norm) is not printed anywhere in the reference tree.
#   turbo2: norm fp16 | qs[32]  (34 B), idx = (qs[j/4] >> ((j%4)*2)) & 3   (the 2-bit half of turbo3)
#   Storage blocks of 32 or 64 values (the fork's QK_TURBO3 / QK_TURBO2 before they became 128,
#   docs/papers/block-size-experiment.md:27-39,270): a vector is 128 / block_values blocks, each norm | qs | signs
#   over its own values with the formulas above taken inside the block (turbo3: 14 B per 32, 26 B per 64; turbo2:
#   10 B, 18 B), and every block of a vector carries the same group norm (block-size-experiment.md:13,45-55).
# --------------------------------------------------------------------------

def fork_block_bytes(bits: int, block_values: int = 128) -> int:
    """Bytes of ONE storage block (of block_values values)."""
    if bits == 4:
        if block_values != 128:
            raise ValueError("turbo4 blocks hold 128 values")
        return 68
    if bits not in (2, 3) or block_values not in (32, 64, 128):
        raise ValueError("no such fork block")
    return 2 + block_values // 4 + (block_values // 8 if bits == 3 else 0)


def fork_row_bytes(bits: int, block_values: int = 128) -> int:
    """Bytes of one 128-value vector: its 128 / block_values storage blocks."""
    return (128 // block_values) * fork_block_bytes(bits, block_values)


def fork_blocks_pack(idx: np.ndarray, g: np.ndarray, bits: int, block_values: int = 128) -> np.ndarray:
    """idx [T,128], g [T] fp16 -> uint8 [T, fork_row_bytes(bits, block_values)], token order."""
    idx = np.asarray(idx).astype(np.uint8)
    T = idx.shape[0]
    gb = np.asarray(g, dtype=np.float16).reshape(T, 1).view(np.uint8)
    if bits == 4:
        out = np.zeros((T, fork_block_bytes(4, block_values)), dtype=np.uint8)
        out[:, 0:2] = gb
        out[:, 4:68] = idx[:, 0::2] | (idx[:, 1::2] << 4)   # bytes 2..3: rnorm, unused, zero
        return out
    bv, bb = block_values, fork_block_bytes(bits, block_values)
    out = np.zeros((T, 128 // bv, bb), dtype=np.uint8)
    for s in range(128 // bv):                              # one storage block after the other
        part = idx[:, s * bv:(s + 1) * bv]
        low = part & 3
        out[:, s, 0:2] = gb
        out[:, s, 2:2 + bv // 4] = low[:, 0::4] | (low[:, 1::4] << 2) | (low[:, 2::4] << 4) | (low[:, 3::4] << 6)
        if bits == 3:
            out[:, s, 2 + bv // 4:] = np.packbits((part >> 2) & 1, axis=1, bitorder="little")
    return out.reshape(T, -1)


def fork_blocks_unpack(buf: np.ndarray, bits: int, block_values: int = 128):
    """-> idx [T,128], g [T] fp16 (the first block's norm; the blocks of a vector all carry the same one)."""
    if bits == 4:
        buf = np.asarray(buf, dtype=np.uint8).reshape(-1, fork_block_bytes(4, block_values))
        T = buf.shape[0]
        g = np.ascontiguousarray(buf[:, 0:2]).view(np.float16).reshape(T)
        j = np.arange(128)
        idx = (buf[:, 4 + j // 2] >> ((j % 2) * 4)) & 0xF
        return idx.astype(np.uint8), g
    bv, bb = block_values, fork_block_bytes(bits, block_values)
    buf = np.asarray(buf, dtype=np.uint8).reshape(-1, 128 // bv, bb)
    T = buf.shape[0]
    g = np.ascontiguousarray(buf[:, 0, 0:2]).view(np.float16).reshape(T)
    j = np.arange(bv)
    idx = np.zeros((T, 128), dtype=np.uint8)
    for s in range(128 // bv):
        blk = buf[:, s]
        part = (blk[:, 2 + j // 4] >> ((j % 4) * 2)) & 3
        if bits == 3:
            part = part | (((blk[:, 2 + bv // 4 + j // 8] >> (j % 8)) & 1) << 2)
        idx[:, s * bv:(s + 1) * bv] = part
    return idx, g


# --------------------------------------------------------------------------
# q8_0-style blocks (textbook ggml; parity unpinned by the reference)
# --------------------------------------------------------------------------

def q8_0_quantize(x):
    """Per 32 consecutive values: scale = max|x|/127 stored as fp16,
    q = roundf(x * (1/scale)) (half away from zero, as ggml's quantize_row_q8_0
    does; scale 0 -> zeros).  All arithmetic in fp32 with the unrounded scale.
    roundf is not floor(|t| + 0.5): for |t| = 0.5 - 2^-25 the sum rounds up to 1.0 in fp32."""
    x = np.asarray(x, dtype=np.float32)
    lead = x.shape[:-1]
    xb = x.reshape(lead + (x.shape[-1] // 32, 32))
    amax = np.abs(xb).max(axis=-1)
    scale = (amax / np.float32(127.0)).astype(np.float32)
    inv = np.where(scale > 0, np.float32(1.0) / np.where(scale > 0, scale, 1), 0).astype(np.float32)
    t = (xb * inv[..., None]).astype(np.float32)
    a = np.abs(t)
    f = np.floor(a)
    q = (np.sign(t) * (f + (a - f >= np.float32(0.5)))).clip(-127, 127).astype(np.int8)  # roundf; a - f is exact
    return q.reshape(x.shape), scale.astype(np.float16)


def q8_0_dequantize(q, scale):
    q = np.asarray(q)
    lead = q.shape[:-1]
    qb = q.reshape(lead + (q.shape[-1] // 32, 32)).astype(np.float64)
    return (qb * np.asarray(scale, dtype=np.float64)[..., None]).reshape(q.shape)


# --------------------------------------------------------------------------
# attention over compressed KV (tests/test_kv_cache.py:73-89,128-131 idiom,
# evaluated in the rotated domain; no reference kernel exists)
# --------------------------------------------------------------------------

def softmax_rows(s):
    """exp(x - max) / sum (tests/test_kv_cache.py:128-131)."""
    e = np.exp(s - s.max(axis=-1, keepdims=True))
    return e / e.sum(axis=-1, keepdims=True)


def decode_attention(q_rot, k_rot, v_rot, scale, n_splits=1, sparse_v_tau=0.0,
                     logit_bias=None, tile=64):
    """One (batch, kv-head) group.

    q_rot [G,128] queries already rotated by the K rotation; k_rot / v_rot
    [N,128] rotated-domain reconstructions (norm * centroid).  Returns the
    rotated-domain output [G,128] (the caller applies the V rotation's
    transpose once), the fraction of (query, position) pairs whose V row was
    skipped, and the fraction with final softmax weight < tau.

    Splits are runs of ceil(ceil(N/tile) / n_splits) tiles of `tile` positions (64; 32 for
    heads of 256 dims, whose tokens take two rows of a 64-row tile).
    Sparse V: within split s the running maximum is the maximum over the
    positions of that split seen so far in tiles of 64; a position's V row is
    skipped for query g when exp(s_i - m_running) < tau.  Softmax statistics
    always include every position.  tau = 0 reproduces the dense result.
    """
    q_rot = np.asarray(q_rot, dtype=np.float64)
    s = scale * (q_rot @ np.asarray(k_rot, dtype=np.float64).T)          # [G,N]
    if logit_bias is not None:
        s = s + logit_bias
    G, N = s.shape
    p_final = softmax_rows(s)
    if sparse_v_tau <= 0.0:
        return p_final @ v_rot, 0.0, 0.0
    n_tiles = -(-N // tile)
    tiles_per_split = -(-n_tiles // n_splits)
    bounds = np.minimum(np.arange(n_splits + 1) * tiles_per_split * tile, N)
    num = np.zeros((G, v_rot.shape[1]))
    den = np.zeros(G)
    m_all = np.full(G, -np.inf)
    skipped = 0
    for a, b in zip(bounds[:-1], bounds[1:]):
        if b <= a:
            continue
        m = np.full(G, -np.inf)
        acc = np.zeros((G, v_rot.shape[1]))
        l = np.zeros(G)
        for c in range(a, b, tile):
            sc = s[:, c:min(c + tile, b)]
            m_new = np.maximum(m, sc.max(axis=1))
            corr = np.exp(m - m_new)
            w = np.exp(sc - m_new[:, None])
            l = l * corr + w.sum(axis=1)
            keep = w >= sparse_v_tau
            skipped += int((~keep).sum())
            acc = acc * corr[:, None] + (w * keep) @ v_rot[c:c + sc.shape[1]]
            m = m_new
        m_new = np.maximum(m_all, m)
        num = num * np.exp(m_all - m_new)[:, None] + acc * np.exp(m - m_new)[:, None]
        den = den * np.exp(m_all - m_new) + l * np.exp(m - m_new)
        m_all = m_new
    return num / den[:, None], skipped / (G * N), float((p_final < sparse_v_tau).mean())


def score_tile(q, k_idx, k_g, centroids, rot_fwd, S, sign_bits, rnorm, qjl_scale):
    """TurboQuant inner-product estimate <q, k_hat> for every (query, key):

      <R q, g * c[idx]>  +  qjl_scale * rnorm * <S q, z>

    (turboquant.py:102-124 with qjl.py:129-132, moved to the rotated /
    projected domain).  rot_fwd maps [n,128] -> rotated; z = +-1 signs."""
    q = np.asarray(q, dtype=np.float64)
    mse = rot_fwd(q) @ turbo_decode_rotated(k_idx, k_g, centroids).T
    corr = (q @ S.T) @ (np.asarray(sign_bits, dtype=np.float64) * (qjl_scale * np.asarray(rnorm, dtype=np.float64))[:, None]).T
    return mse + corr
