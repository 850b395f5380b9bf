"""Production ("turbo2/3/4") KV format on the GPU: head_dim 128, sign-diagonal
WHT rotation, Lloyd-Max codes packed in 128-token blocks with a corrected fp16
norm per vector, and attention computed directly on the packed buffers.

The reference describes this format only in its docs (block layout
docs/papers/block-size-experiment.md:33-39, write-side norm correction
benchmarks/temporal_decay_prototype.py:58-90, pre-rotated queries
docs/pre-rotate-queries-plan.md:5-8, Sparse V docs/papers/sparse-v-dequant.md:66-78);
its arithmetic is the MSE-only quantiser of turboquant/polar_quant.py:56-119
with the rotation of turboquant/rotation.py:163-185.

All tensors are torch CUDA tensors used as plain buffers; NumPy inputs are
copied to the device first.
"""
from __future__ import annotations

import ctypes as C
import math
import os

import numpy as np

from . import _lib as L
from .codebook import optimal_centroids
from .qjl import projection_matrix
from .rotation import random_rotation_fast

HEAD_DIM = 128
BLOCK_TOKENS = 128


def packed_bytes(bits: int, n_seqs: int, tokens: int) -> int:
    n = L.lib().tq_packed_bytes(bits, n_seqs, tokens)
    if n < 0:
        raise ValueError("bits must be 2, 3 or 4 and sizes non-negative")
    return int(n)


# Centroid tables the llama.cpp fork ships (d = 128), as printed in the reference's documents:
# 2- and 3-bit benchmarks/temporal_decay_prototype.py:38-46, 4-bit docs/papers/turbo4-resurrection.md:163-166.
# TurboCodec(bits, centroids=PRODUCTION_CENTROIDS[bits]) makes caches interchangeable with it.
PRODUCTION_CENTROIDS = {
    2: np.array([-0.133462, -0.039994, 0.039994, 0.133462]),
    3: np.array([-0.190685, -0.117832, -0.065717, -0.021460, 0.021460, 0.065717, 0.117832, 0.190685]),
    4: np.array([-0.1739, -0.1172, -0.0895, -0.0688, -0.0513, -0.0356, -0.0210, -0.0069,
                 0.0069, 0.0210, 0.0356, 0.0513, 0.0688, 0.0895, 0.1172, 0.1739]),
}


class TurboCodec:
    """One quantiser (rotation signs + codebook [+ QJL projection]) for K or V.

    seed / single_diagonal: signs1, signs2 = the two `choice` draws of
        random_rotation_fast(128, default_rng(seed)); single_diagonal forces
        signs2 to ones (one sign diagonal, as in BASELINE config 1).
    centroids: table override (default optimal_centroids(bits, 128)).
    projection: None | "orthogonal" | "gaussian" with projection_seed: enables
        store_qjl / score_tile.
    """

    def __init__(self, bits: int = 3, seed: int = 42, *, single_diagonal: bool = False, centroids=None,
                 norm_correction: bool = True, projection: str | None = None, projection_seed: int | None = None,
                 signs1=None, signs2=None):
        if bits not in (2, 3, 4):
            raise ValueError(f"turbo format supports 2, 3 or 4 bits, got {bits}")
        self.bits = bits
        self.d = HEAD_DIM
        if signs1 is None:
            signs1, s2, _ = random_rotation_fast(HEAD_DIM, np.random.default_rng(seed))
            signs2 = np.ones(HEAD_DIM) if single_diagonal else s2
        self.signs1 = np.asarray(signs1, dtype=np.float64)
        self.signs2 = np.asarray(signs2, dtype=np.float64)
        self.centroids = optimal_centroids(bits, HEAD_DIM) if centroids is None else np.asarray(centroids, np.float64)
        if self.centroids.shape != (1 << bits,):
            raise ValueError(f"centroids must have {1 << bits} entries")
        self.norm_correction = norm_correction
        self.S = None
        self.projection_scale = 0.0
        if projection is not None:
            self.S, self.projection_scale = projection_matrix(
                HEAD_DIM, seed + 1000 if projection_seed is None else projection_seed, projection)
        self._handle = None

    @property
    def handle(self) -> L.Handle:
        if self._handle is None:
            self._handle = L.Handle(HEAD_DIM, self.bits, self.centroids, signs1=self.signs1, signs2=self.signs2,
                                    projection=self.S, projection_scale=self.projection_scale,
                                    norm_correction=self.norm_correction)
        return self._handle

    # ---- store / load ---------------------------------------------------------
    @staticmethod
    def _as_seqs(x):
        xd = L.to_device(x)
        if xd.shape[-1] != HEAD_DIM:
            raise ValueError(f"last dimension must be {HEAD_DIM}, got {xd.shape[-1]}")
        if xd.dim() == 2:
            xd = xd[None]
        tokens = xd.shape[-2]
        n_seqs = xd.numel() // (tokens * HEAD_DIM) if tokens else 0
        return xd.reshape(n_seqs, tokens, HEAD_DIM), n_seqs, tokens

    def store(self, x, kind: str = "k", out=None):
        """x [..., tokens, 128] (fp16/fp32/fp64) -> packed uint8 buffer; every
        leading index is a sequence whose blocks do not mix with others."""
        tt = L.torch()
        xd, n_seqs, tokens = self._as_seqs(x)
        nbytes = packed_bytes(self.bits, n_seqs, tokens)
        if out is None:
            out = tt.empty(nbytes, dtype=tt.uint8, device=xd.device)
        elif out.numel() < nbytes:
            raise ValueError(f"out holds {out.numel()} bytes, need {nbytes}")
        elif n_seqs > 1 and out.numel() != nbytes:
            # sequences are laid out ceil(tokens / 128) blocks apart: a buffer sized for a larger capacity has
            # another stride, and every sequence after the first would land in the wrong place
            raise ValueError(f"out holds {out.numel()} bytes but {n_seqs} sequences of {tokens} tokens take exactly "
                             f"{nbytes}; fill a cache laid out for a larger capacity with append()")
        L.check(L.lib().tq_store(self.handle.h, L.ptr(xd), n_seqs, tokens, L.dtype_code(xd),
                                 L.KIND_K if kind == "k" else L.KIND_V, L.ptr(out), L.stream_ptr()))
        return out

    def store_kv(self, v_codec: "TurboCodec", k, v, out_k=None, out_v=None, capacity: int | None = None):
        """K with this codec and V with `v_codec` in one launch -> (packed_k, packed_v);
        the same bytes as store(k, "k") and v_codec.store(v, "v").

        capacity: prefill of a growing cache (tq_store_kv_cache): out_k / out_v are buffers of
        packed_bytes(bits, n_seqs, capacity) bytes, the layout of append_kv() and DecodeAttention(capacity=...),
        and every sequence's tokens go to its first blocks."""
        tt = L.torch()
        kd, n_seqs, tokens = self._as_seqs(k)
        vd, n_seqs_v, tokens_v = v_codec._as_seqs(v)
        if (n_seqs, tokens) != (n_seqs_v, tokens_v) or kd.dtype != vd.dtype:
            raise ValueError("k and v must have the same shape and dtype")
        if capacity is not None:
            if tokens > capacity:
                raise ValueError(f"{tokens} tokens do not fit a capacity of {capacity}")
            if out_k is None or out_v is None:
                raise ValueError("prefill needs the cache buffers (out_k, out_v)")
            nk, nv = packed_bytes(self.bits, n_seqs, capacity), packed_bytes(v_codec.bits, n_seqs, capacity)
            if out_k.numel() != nk or out_v.numel() != nv:
                raise ValueError(f"cache buffers hold {out_k.numel()} and {out_v.numel()} bytes, a capacity of {capacity} "
                                 f"tokens for {n_seqs} sequences takes {nk} and {nv}")
            L.check(L.lib().tq_store_kv_cache(self.handle.h, v_codec.handle.h, L.ptr(kd), L.ptr(vd), n_seqs, tokens, capacity,
                                              L.dtype_code(kd), L.ptr(out_k), L.ptr(out_v), L.stream_ptr()))
            return out_k, out_v
        nk, nv = packed_bytes(self.bits, n_seqs, tokens), packed_bytes(v_codec.bits, n_seqs, tokens)
        pk = tt.empty(nk, dtype=tt.uint8, device=kd.device) if out_k is None else out_k
        pv = tt.empty(nv, dtype=tt.uint8, device=kd.device) if out_v is None else out_v
        if pk.numel() < nk or pv.numel() < nv:
            raise ValueError(f"output buffers hold {pk.numel()} and {pv.numel()} bytes, need {nk} and {nv}")
        if n_seqs > 1 and (pk.numel() != nk or pv.numel() != nv):
            raise ValueError(f"output buffers hold {pk.numel()} and {pv.numel()} bytes but {n_seqs} sequences of "
                             f"{tokens} tokens take exactly {nk} and {nv}; fill a cache laid out for a larger "
                             "capacity with store_kv(capacity=...) or append_kv()")
        L.check(L.lib().tq_store_kv(self.handle.h, v_codec.handle.h, L.ptr(kd), L.ptr(vd), n_seqs, tokens,
                                    L.dtype_code(kd), L.ptr(pk), L.ptr(pv), L.stream_ptr()))
        return pk, pv

    def append(self, x, packed, pos, capacity: int, kind: str = "k", overrun=None):
        """Write the tokens x [n_seqs, n_new, 128] at positions pos .. pos+n_new-1 of
        `packed`, a buffer of packed_bytes(bits, n_seqs, capacity) bytes (tq_append).  pos: an int, or an int64
        device tensor with one element that holds the position when the launch runs (tq_append_at); with such a
        position, `overrun` (a zeroed int32 device tensor with one element) collects OVERRUN_* bits when a launch
        finds a position that it refuses, see overrun_bits()."""
        xd, n_seqs, n_new = self._as_seqs(x)
        need = packed_bytes(self.bits, n_seqs, capacity)
        if packed.numel() < need:
            raise ValueError(f"packed holds {packed.numel()} bytes, need {need}")
        if _position_on_device(pos):
            L.check(L.lib().tq_append_at(self.handle.h, L.ptr(xd), n_seqs, L.ptr(pos), n_new, capacity, L.dtype_code(xd),
                                         L.KIND_K if kind == "k" else L.KIND_V, L.ptr(packed), _overrun_ptr(overrun),
                                         L.stream_ptr()))
            return packed
        L.check(L.lib().tq_append(self.handle.h, L.ptr(xd), n_seqs, pos, n_new, capacity, L.dtype_code(xd),
                                  L.KIND_K if kind == "k" else L.KIND_V, L.ptr(packed), L.stream_ptr()))
        return packed

    def append_kv(self, v_codec: "TurboCodec", k, v, packed_k, packed_v, pos, capacity: int, overrun=None):
        """append() of the K tokens (this codec) and the V tokens (`v_codec`) of one decode step
        in one launch (tq_append_kv).  pos: an int, or an int64 device tensor with one element that holds the
        position when the launch runs (tq_append_kv_at: a captured step replayed while the cache grows; `overrun`
        as in append())."""
        kd, n_seqs, n_new = self._as_seqs(k)
        vd, vs, vn = self._as_seqs(v)
        if (vs, vn) != (n_seqs, n_new) or vd.dtype != kd.dtype:
            raise ValueError("k and v must have the same shape and dtype")
        for codec, buf in ((self, packed_k), (v_codec, packed_v)):
            need = packed_bytes(codec.bits, n_seqs, capacity)
            if buf.numel() < need:
                raise ValueError(f"packed holds {buf.numel()} bytes, need {need}")
        if _position_on_device(pos):
            L.check(L.lib().tq_append_kv_at(self.handle.h, v_codec.handle.h, L.ptr(kd), L.ptr(vd), n_seqs, L.ptr(pos), n_new,
                                            capacity, L.dtype_code(kd), L.ptr(packed_k), L.ptr(packed_v),
                                            _overrun_ptr(overrun), L.stream_ptr()))
            return packed_k, packed_v
        L.check(L.lib().tq_append_kv(self.handle.h, v_codec.handle.h, L.ptr(kd), L.ptr(vd), n_seqs, pos, n_new, capacity,
                                     L.dtype_code(kd), L.ptr(packed_k), L.ptr(packed_v), L.stream_ptr()))
        return packed_k, packed_v

    def requantize_to(self, dst_codec: "TurboCodec", packed, n_seqs: int, tokens: int, kind: str = "k"):
        """Temporal decay: re-quantise a buffer written with this codec to the narrower
        `dst_codec` (same rotation) -> new packed buffer (tq_requantize)."""
        tt = L.torch()
        if not (np.array_equal(self.signs1, dst_codec.signs1) and np.array_equal(self.signs2, dst_codec.signs2)):
            raise ValueError("requantize_to: both codecs must use the same rotation (same sign diagonals); "
                             "codes written under one rotation mean nothing under another")
        out = tt.empty(packed_bytes(dst_codec.bits, n_seqs, tokens), dtype=tt.uint8, device=packed.device)
        L.check(L.lib().tq_requantize(self.handle.h, dst_codec.handle.h, L.ptr(packed), n_seqs, tokens,
                                      L.KIND_K if kind == "k" else L.KIND_V, L.ptr(out), L.stream_ptr()))
        return out

    def export_fork_blocks(self, packed, n_seqs: int, tokens: int, kind: str = "k", block_values: int = 128):
        """-> uint8 [n_seqs, tokens, row bytes]: the llama.cpp fork's block layout, 50 | 68 | 34 bytes per vector with
        the fork's present 128-value storage blocks; block_values = 32 or 64 gives the layout of its earlier builds
        (2- and 3-bit rows: four blocks of 14 | 10 bytes, two of 26 | 18; docs/papers/block-size-experiment.md:27-39)."""
        tt = L.torch()
        fb = int(L.lib().tq_fork_row_bytes(self.bits, block_values))
        if fb < 0:
            raise ValueError(f"the fork has no {self.bits}-bit layout with {block_values} values per storage block")
        out = tt.empty((n_seqs, tokens, fb), dtype=tt.uint8, device=packed.device)
        L.check(L.lib().tq_export_fork_blocks_sized(self.handle.h, L.ptr(packed), n_seqs, tokens,
                                                    L.KIND_K if kind == "k" else L.KIND_V, block_values, L.ptr(out),
                                                    L.stream_ptr()))
        return out

    def import_fork_blocks(self, blocks, kind: str = "k", block_values: int = 128):
        """Fork blocks [n_seqs, tokens, row bytes of this width and block size] -> packed buffer of this library."""
        tt = L.torch()
        dev = L.require_gpu()
        bd = blocks if isinstance(blocks, tt.Tensor) else tt.from_numpy(np.ascontiguousarray(blocks))
        fb = int(L.lib().tq_fork_row_bytes(self.bits, block_values))
        if fb < 0:
            raise ValueError(f"the fork has no {self.bits}-bit layout with {block_values} values per storage block")
        if bd.dtype != tt.uint8 or bd.dim() != 3 or bd.shape[2] != fb:
            raise ValueError("blocks must be uint8 [n_seqs, tokens, row bytes of this width and block size]")
        bd = bd.to(dev)
        n_seqs, tokens = int(bd.shape[0]), int(bd.shape[1])
        out = tt.empty(packed_bytes(self.bits, n_seqs, tokens), dtype=tt.uint8, device=bd.device)
        L.check(L.lib().tq_import_fork_blocks_sized(self.handle.h, L.ptr(bd.contiguous()), n_seqs, tokens,
                                                    L.KIND_K if kind == "k" else L.KIND_V, block_values, L.ptr(out),
                                                    L.stream_ptr()))
        return out

    def store_qjl(self, x):
        """K-layout codes plus the residual sign sketch -> (packed, sign_bits [n,16] uint8, rnorms [n] fp16)."""
        tt = L.torch()
        xd, n_seqs, tokens = self._as_seqs(x)
        n = n_seqs * tokens
        packed = tt.empty(packed_bytes(self.bits, n_seqs, tokens), dtype=tt.uint8, device=xd.device)
        bits = tt.empty((n, 16), dtype=tt.uint8, device=xd.device)
        rn = tt.empty((n,), dtype=tt.float16, device=xd.device)
        L.check(L.lib().tq_store_qjl(self.handle.h, L.ptr(xd), n_seqs, tokens, L.dtype_code(xd), L.ptr(packed),
                                     L.ptr(bits), L.ptr(rn), L.stream_ptr()))
        return packed, bits, rn

    def load(self, packed, n_seqs: int, tokens: int, kind: str = "k", domain: str = "original", dtype=None, out=None):
        """packed -> [n_seqs, tokens, 128] values in the original or the rotated domain (into `out` if given)."""
        tt = L.torch()
        if out is None:
            dtype = tt.float32 if dtype is None else dtype
            out = tt.empty((n_seqs, tokens, HEAD_DIM), dtype=dtype, device=packed.device)
        elif out.numel() != n_seqs * tokens * HEAD_DIM or not out.is_contiguous():
            raise ValueError(f"out must be a contiguous tensor of {n_seqs * tokens * HEAD_DIM} elements")
        L.check(L.lib().tq_load(self.handle.h, L.ptr(packed), n_seqs, tokens, L.KIND_K if kind == "k" else L.KIND_V,
                                L.ptr(out), L.dtype_code(out),
                                L.DOMAIN_ORIGINAL if domain == "original" else L.DOMAIN_ROTATED, L.stream_ptr()))
        return out

    def load_kv(self, v_codec: "TurboCodec", packed_k, packed_v, n_seqs: int, tokens: int, out_k=None, out_v=None):
        """(packed_k, packed_v) -> K and V [n_seqs, tokens, 128] fp16 in the original domain in one launch;
        the same values as load(packed_k, .., "k", dtype=float16) and v_codec.load(packed_v, .., "v", dtype=float16)."""
        tt = L.torch()
        outs = []
        for o in (out_k, out_v):
            if o is None:
                o = tt.empty((n_seqs, tokens, HEAD_DIM), dtype=tt.float16, device=packed_k.device)
            elif o.dtype != tt.float16 or o.numel() != n_seqs * tokens * HEAD_DIM or not o.is_contiguous():
                raise ValueError(f"outputs must be contiguous fp16 tensors of {n_seqs * tokens * HEAD_DIM} elements")
            outs.append(o)
        nk, nv = packed_bytes(self.bits, n_seqs, tokens), packed_bytes(v_codec.bits, n_seqs, tokens)
        if packed_k.numel() < nk or packed_v.numel() < nv:
            raise ValueError(f"packed buffers hold {packed_k.numel()} and {packed_v.numel()} bytes, need {nk} and {nv}")
        L.check(L.lib().tq_load_kv(self.handle.h, v_codec.handle.h, L.ptr(packed_k), L.ptr(packed_v), n_seqs, tokens,
                                   L.ptr(outs[0]), L.ptr(outs[1]), L.stream_ptr()))
        return outs[0], outs[1]

    def unpack_codes(self, packed, n_seqs: int, tokens: int, kind: str = "k"):
        """packed -> (indices uint8 [n_seqs, tokens, 128], stored norms fp32 [n_seqs, tokens])."""
        tt = L.torch()
        idx = tt.empty((n_seqs, tokens, HEAD_DIM), dtype=tt.uint8, device=packed.device)
        norms = tt.empty((n_seqs, tokens), dtype=tt.float32, device=packed.device)
        L.check(L.lib().tq_unpack_codes(self.handle.h, L.ptr(packed), n_seqs, tokens,
                                        L.KIND_K if kind == "k" else L.KIND_V, L.ptr(idx), L.ptr(norms),
                                        L.stream_ptr()))
        return idx, norms

    def rotate(self, x, transpose: bool = False, dtype=None):
        """R x (or R^T x) with the one-wavefront-per-vector fp32 butterfly."""
        tt = L.torch()
        xd = L.to_device(x)
        if xd.dtype == tt.float64:
            xd = xd.to(tt.float32)
        flat = xd.reshape(-1, HEAD_DIM)
        out = tt.empty(flat.shape, dtype=xd.dtype if dtype is None else dtype, device=xd.device)
        L.check(L.lib().tq_rotate(self.handle.h, L.ptr(flat), L.ptr(out), flat.shape[0], L.dtype_code(flat),
                                  L.dtype_code(out), int(transpose), L.stream_ptr()))
        return out.reshape(xd.shape)

    # ---- prefill-shaped inner-product estimator --------------------------------
    def score_tile(self, q, packed, sign_bits, rnorms, n_keys: int, out_dtype=None, store: bool = True, out=None):
        """logits [nq, n_keys] = <R q, g c[idx]> + scale * rnorm * <S q, z>.  store=False runs the
        computation without writing the logits (a measurement aid) and returns None.  out: a
        contiguous [nq, n_keys] tensor of the output type to write into instead of a new one."""
        tt = L.torch()
        qd = L.to_device(q).reshape(-1, HEAD_DIM)
        nq = qd.shape[0]
        if out is not None:
            out_dtype = out.dtype
        out_dtype = tt.float32 if out_dtype is None else out_dtype
        if out_dtype not in (tt.float32, tt.float16):
            raise TypeError(f"logits must be float32 or float16, not {out_dtype}")
        if out is not None:
            if tuple(out.shape) != (nq, n_keys) or not out.is_contiguous() or not out.is_cuda:
                raise ValueError(f"out must be a contiguous device tensor of shape ({nq}, {n_keys})")
            logits = out
        else:
            logits = tt.empty((nq, n_keys), dtype=out_dtype, device=qd.device) if store else None
        ws = tt.empty(max((nq + 31) // 32 * 32 * 512, 16), dtype=tt.uint8, device=qd.device)
        L.check(L.lib().tq_score_tile(self.handle.h, L.ptr(qd), L.dtype_code(qd), nq, L.ptr(packed), L.ptr(sign_bits),
                                      L.ptr(rnorms), n_keys, L.ptr(logits) if store else None,
                                      L.TQ_F16 if out_dtype == tt.float16 else L.TQ_F32,
                                      L.ptr(ws), ws.numel(), L.stream_ptr()))
        return logits


def _kind_name(kind: str) -> str:
    if kind not in ("k", "v"):
        raise ValueError(f"kind must be 'k' or 'v', got {kind!r}")
    return kind


def q8_0_store(x, kind: str = "k"):
    """x [..., tokens, 128] -> q8_0-style buffer (uint8), n_seqs, tokens.  kind="v" lays the same int8
    values and scales out as the decode kernel reads V rows (dim-major inside 64-token tiles)."""
    tt = L.torch()
    xd, n_seqs, tokens = TurboCodec._as_seqs(x)
    out = tt.empty(int(L.lib().tq_q8_0_bytes(n_seqs, tokens)), dtype=tt.uint8, device=xd.device)
    fn = L.lib().tq_q8_0_store if _kind_name(kind) == "k" else L.lib().tq_q8_0_store_v
    L.check(fn(L.ptr(xd), n_seqs, tokens, L.dtype_code(xd), L.ptr(out), L.stream_ptr()))
    return out, n_seqs, tokens


def _position_on_device(pos) -> bool:
    """False for a host integer; True for an int64 device tensor with one element (anything else raises)."""
    if isinstance(pos, (int, np.integer)):
        return False
    tt = L.torch()
    if not isinstance(pos, tt.Tensor) or pos.dtype != tt.int64 or not pos.is_cuda or pos.numel() != 1:
        raise ValueError("a position on the device must be an int64 device tensor with one element")
    return True


OVERRUN_NEGATIVE, OVERRUN_NO_ROOM = 1, 2   # TQ_OVERRUN_* of include/tq.h


def _overrun_ptr(overrun):
    """NULL, or the address of the caller's sticky overrun word (int32 device tensor with one element)."""
    if overrun is None:
        return None
    tt = L.torch()
    if not isinstance(overrun, tt.Tensor) or overrun.dtype != tt.int32 or not overrun.is_cuda or overrun.numel() != 1:
        raise ValueError("overrun must be an int32 device tensor with one element")
    return L.ptr(overrun)


def overrun_bits(overrun) -> int:
    """Read the overrun word of the *_at appends (synchronises): 0, or OVERRUN_NEGATIVE | OVERRUN_NO_ROOM bits of
    the launches that refused their position since the word was last cleared."""
    return int(overrun.item())


def q8_0_append(x, packed, pos, capacity: int, kind: str = "k", overrun=None):
    """Write the tokens x [n_seqs, n_new, 128] at positions pos .. pos+n_new-1 of a q8_0-style buffer laid
    out for `capacity` tokens per sequence (zero-initialised; tq_q8_0_append).  pos: an int, or an int64 device
    tensor with one element read when the launch runs (tq_q8_0_append_at; `overrun` as in TurboCodec.append)."""
    xd, n_seqs, n_new = TurboCodec._as_seqs(x)
    need = int(L.lib().tq_q8_0_bytes(n_seqs, capacity))
    if packed.numel() < need:
        raise ValueError(f"packed holds {packed.numel()} bytes, need {need}")
    if _position_on_device(pos):
        L.check(L.lib().tq_q8_0_append_at(L.ptr(xd), n_seqs, L.ptr(pos), n_new, capacity, L.dtype_code(xd),
                                          L.KIND_K if _kind_name(kind) == "k" else L.KIND_V, L.ptr(packed),
                                          _overrun_ptr(overrun), L.stream_ptr()))
        return packed
    L.check(L.lib().tq_q8_0_append(L.ptr(xd), n_seqs, pos, n_new, capacity, L.dtype_code(xd),
                                   L.KIND_K if _kind_name(kind) == "k" else L.KIND_V, L.ptr(packed), L.stream_ptr()))
    return packed


def q8_0_unpack(packed, n_seqs: int, tokens: int, kind: str = "k"):
    """int8 values [n_seqs, tokens, 128] and fp32 scales [n_seqs, tokens, 4] of a q8_0_store buffer."""
    tt = L.torch()
    q = tt.empty((n_seqs, tokens, HEAD_DIM), dtype=tt.int8, device=packed.device)
    s = tt.empty((n_seqs, tokens, 4), dtype=tt.float32, device=packed.device)
    fn = L.lib().tq_q8_0_unpack if _kind_name(kind) == "k" else L.lib().tq_q8_0_unpack_v
    L.check(fn(L.ptr(packed), n_seqs, tokens, L.ptr(q), L.ptr(s), L.stream_ptr()))
    return q, s


class DecodeAttention:
    """softmax(scale * q k^T) v over packed K/V; n_q_heads a multiple of n_kv_heads.

    The kernels take four query heads of a KV head per pass over its K/V, or
    eight when the group has more than four, so groups of up to 8 read the cache
    once and a group of G > 8 reads it ceil(G / 8) times.

    Holds the parameter block and the split workspace so that repeated steps
    allocate nothing.  K is a turbo buffer (k_codec given) or a q8_0-style
    buffer (k_codec None); V is a turbo buffer written with kind="v" (v_codec
    given) or a q8_0_store(x, kind="v") buffer (v_codec None).
    """

    def __init__(self, k_codec: TurboCodec | None, v_codec: TurboCodec | None, batch: int, n_q_heads: int, n_kv_heads: int,
                 tokens: int, *, n_splits: int | None = None, scale: float | None = None, sparse_v_tau: float = 0.0,
                 capacity: int = 0, tokens_on_device=None, poison_output: bool | None = None, head_dim: int = HEAD_DIM):
        """tokens_on_device: an int64 device tensor (one element) that holds the context length when a call runs;
        `tokens` is then the largest length it may take.  One captured launch (HIP graph) can so be replayed while
        the cache grows; Sparse V is not available in this mode.
        poison_output (default: on when the environment holds TQ_POISON_OUTPUT=1): fill the output rows with NaN
        before every call, so that a row the launch did not write - the split partials are merged inside the launch by
        whichever workgroup of a group finishes last - shows as NaN instead of the previous call's values.  A debug
        aid: one small fill kernel per call.
        head_dim: 128, or 256 - a head's vector as two 128-value groups, each rotated, quantised and normed by itself
        (the fork's 128-value blocks, docs/getting-started.md:68).  The caches are then those of 128-dim heads with
        two rows per token: rows_of_256(x) gives the [n, 2 * tokens, 128] view that store / append / load take, and
        `tokens`, `capacity`, `pos` of those calls count rows (2 * tokens).  Turbo K at least as wide as turbo V, or
        q8_0-style rows on either side."""
        tt = L.torch()
        dev = L.require_gpu()
        self.k_codec, self.v_codec = k_codec, v_codec
        if head_dim not in (HEAD_DIM, 2 * HEAD_DIM):
            raise ValueError(f"head_dim {head_dim}: the packed-cache kernels take 128 or 256")
        self.head_dim = head_dim
        if n_splits is None:
            n_splits = default_splits(batch * n_kv_heads, tokens * (head_dim // HEAD_DIM),
                                      eight_heads=head_dim == HEAD_DIM and n_q_heads // max(n_kv_heads, 1) > 4,
                                      turbo_rows=k_codec is not None and v_codec is not None,
                                      one_workgroup_per_cu=v_codec is None or (head_dim != HEAD_DIM and k_codec is None))
        self.params = L.TQAttnParams(batch=batch, n_q_heads=n_q_heads, n_kv_heads=n_kv_heads, tokens=tokens,
                                     capacity=capacity, n_splits=n_splits, k_format=L.KFMT_TURBO if k_codec is not None else L.KFMT_Q8_0,
                                     v_format=L.KFMT_TURBO if v_codec is not None else L.KFMT_Q8_0,
                                     scale=(1.0 / math.sqrt(head_dim)) if scale is None else scale,
                                     sparse_v_tau=sparse_v_tau, head_dim=head_dim)
        self.tokens_on_device = tokens_on_device   # kept alive with the object
        if tokens_on_device is not None:
            if tokens_on_device.dtype != tt.int64 or not tokens_on_device.is_cuda or tokens_on_device.numel() != 1:
                raise ValueError("tokens_on_device must be an int64 device tensor with one element")
            if sparse_v_tau > 0:
                raise ValueError("Sparse V keeps no count for a context length read from device memory")
            self.params.tokens_dev = tokens_on_device.data_ptr()
        nbytes = L.lib().tq_attn_workspace_bytes(C.byref(self.params))
        if nbytes < 0:
            L.check(L.ERR_ARG)
        self.workspace = tt.empty(int(nbytes), dtype=tt.uint8, device=dev)
        self.skip = tt.zeros(2, dtype=tt.int64, device=dev)
        self.out = tt.empty((batch, n_q_heads, head_dim), dtype=tt.float32, device=dev)
        self.poison_output = os.environ.get("TQ_POISON_OUTPUT", "0") == "1" if poison_output is None else bool(poison_output)

    def __call__(self, q, k_packed, v_packed, bias=None, sparse_bias=None):
        """q [batch, n_q_heads, 128] in the original domain -> out fp32 [batch, n_q_heads, 128].
        bias: dense additive logit bias [batch, n_q_heads, tokens] fp32.  sparse_bias: (positions, values), int32 and fp32
        device tensors [batch, n_q_heads, E]: a bias that is zero except at E positions per head, positions ascending
        within a head and unique (sparse_bias_from_dense() builds the pair); both may be given and add up."""
        qd = L.to_device(q)
        if self.poison_output:
            self.out.fill_(float("nan"))
        tt = L.torch()
        if sparse_bias is not None:
            pos, val = sparse_bias
            want = (self.params.batch, self.params.n_q_heads)
            if (pos.dtype != tt.int32 or val.dtype != tt.float32 or not pos.is_cuda or not val.is_cuda or pos.dim() != 3
                    or tuple(pos.shape[:2]) != want or pos.shape != val.shape):
                raise ValueError("sparse_bias must be (int32 positions, float32 values), device tensors [batch, n_q_heads, E]")
            pos, val = pos.contiguous(), val.contiguous()
            self.params.bias_entries = int(pos.shape[2])
            self.params.bias_pos, self.params.bias_val = pos.data_ptr(), val.data_ptr()
            self._sparse_bias = (pos, val)   # kept alive until the next call
        else:
            self.params.bias_entries = 0
            self.params.bias_pos = self.params.bias_val = None
        hk = self.k_codec.handle.h if self.k_codec is not None else None
        hv = self.v_codec.handle.h if self.v_codec is not None else None
        L.check(L.lib().tq_decode_attention(hk, hv, C.byref(self.params), L.ptr(qd),
                                            L.dtype_code(qd), L.ptr(k_packed), None, L.ptr(v_packed), L.ptr(bias),
                                            L.ptr(self.out),
                                            L.ptr(self.skip if self.params.sparse_v_tau > 0 else None),
                                            L.ptr(self.workspace),
                                            self.workspace.numel(), L.stream_ptr()))
        return self.out

    def set_tokens(self, tokens: int) -> None:
        """Context length of the next calls (a cache that grows by append); the
        buffers stay laid out for `capacity` tokens per sequence."""
        if self.params.capacity and tokens > self.params.capacity:
            raise ValueError(f"tokens {tokens} exceed the capacity {self.params.capacity}")
        self.params.tokens = tokens

    def skip_rate(self) -> float:
        s = self.skip.cpu().numpy()
        return float(s[0]) / float(s[1]) if s[1] else 0.0


def rows_of_256(x):
    """[n, tokens, 256] -> the [n, 2 * tokens, 128] view of the same memory: row 2 * token + half holds dims
    128 * half .. 128 * half + 127 of the token, the unit that the store, append and load calls work on for heads of
    256 dims (no copy; x must be contiguous)."""
    if x.shape[-1] != 2 * HEAD_DIM:
        raise ValueError(f"last dimension {x.shape[-1]}, expected {2 * HEAD_DIM}")
    if hasattr(x, "is_contiguous") and not x.is_contiguous():
        raise ValueError("rows_of_256 needs a contiguous tensor")
    return x.reshape(*x.shape[:-2], 2 * x.shape[-2], HEAD_DIM)


def sparse_bias_from_dense(bias, max_entries: int | None = None):
    """Dense logit bias [batch, n_q_heads, tokens] -> (positions int32, values fp32) [batch, n_q_heads, E] holding its
    non-zero entries, positions ascending within a head and lists padded with position 2^31 - 1 (value 0).  E is the
    largest count of non-zero entries over the heads (ValueError if that exceeds max_entries)."""
    tt = L.torch()
    bd = L.to_device(bias).to(tt.float32)
    nz = bd != 0
    e = int(nz.sum(dim=-1).max().item()) if bd.numel() else 0
    if max_entries is not None and e > max_entries:
        raise ValueError(f"a head has {e} non-zero bias entries, more than {max_entries}")
    e = max(e, 1)
    # a stable sort of "is zero" puts every head's non-zero positions first, in ascending order
    order = tt.sort((~nz).to(tt.int8), dim=-1, stable=True).indices[..., :e]
    val = tt.gather(bd, -1, order)
    pos = tt.where(val != 0, order, tt.full_like(order, 2 ** 31 - 1)).to(tt.int32)
    return pos.contiguous(), val.contiguous()


def default_splits(n_groups: int, tokens: int, eight_heads: bool = False, turbo_rows: bool = True,
                   one_workgroup_per_cu: bool = False) -> int:
    """Context splits per (batch, kv head): one wavefront per split.  A large step (eight or more 64-token tiles
    per wavefront at four wavefronts per SIMD on 256 CUs x 4 SIMDs) gets those 4096 wavefronts; a smaller one is
    bound by what a workgroup does once (tables, queries, the merge of its wavefronts' partials) and measured faster
    on 2048 wavefronts, i.e. one workgroup of eight per CU (four sequences at 32K: 25.7 against 27.1 us; one at 128K:
    27.6 against 30.2 us), down to two tiles per split (one sequence at 32K: 15.5 us; one tile per split 18.6 us).
    The kernel groups up to 16 splits (the largest power of two dividing the count) into one workgroup, so the count
    is rounded down to a multiple of 16, or to a power of two below 16.
    eight_heads: more than four query heads per KV head (128-dim heads).  That variant's registers leave room for one
    workgroup per CU, so one round of 256 workgroups is the aim: twelve wavefronts each (a split count that is a
    multiple of 12; turbo K and V rows) when a wavefront then still has twenty tiles, eight otherwise (16 sequences x 8
    KV heads at 32K, 64 query heads: 94.6 us with 24 splits, 97.9 with 16, 104.8 with 32; 8 sequences: 51.5 us with 32
    splits, 52.0 with 48, 64.6 with 64).
    one_workgroup_per_cu: the other variants whose workgroups of eight wavefronts fit a CU once (q8_0-style V rows; 256-dim
    heads with q8_0-style rows on either side): 2048 wavefronts, one round of workgroups (16 x 8 groups at 32K, turbo3 K
    with q8_0-style V: 120.5 us with 16 splits against 124.9 with 32; 256-dim heads, q8_0-style K with turbo3 V: 123.2
    against 130.1; with Sparse V the same or more)."""
    tiles = max(1, (tokens + 63) // 64)
    total = n_groups * tiles
    if eight_heads:
        if turbo_rows and total >= 20 * 3072 and 3072 // n_groups >= 12:
            n = min(3072 // n_groups, tiles // 2) // 12 * 12
            if n >= 12:
                return n
        waves = 2048
    elif one_workgroup_per_cu:
        waves = 2048
    else:
        waves = 4096 if total >= 8 * 4096 else 2048
    want = max(1, (waves + n_groups - 1) // n_groups)
    n = int(max(1, min(want, tiles // 2 if tiles >= 2 else 1)))
    if n >= 16:
        return n // 16 * 16
    return 1 << (n.bit_length() - 1)
