"""Per-layer cache formats: which layers keep K / V as q8_0 and which as turboN.

The reference describes these policies for its llama.cpp fork, where the
TURBO_LAYER_ADAPTIVE environment variable selects one (no Python code exists):
  mode 0  uniform base formats                         (docs/experiment-layer-adaptive.md:10)
  mode 1  q8_0 K and V on the first and last 4 layers  (docs/experiment-layer-adaptive.md:11)
  mode 2  q8_0 K and V on the last 8 layers            (docs/experiment-layer-adaptive.md:12)
  mode 5  turbo4 V on the first 2 and last 2 layers    (docs/papers/layer-aware-v-compression.md:83)
  mode 6  turbo4 V on the last 8 layers                (docs/papers/layer-aware-v-compression.md:84)
  mode 7  "Boundary V": q8_0 V on the first 2 and last 2 layers, K unchanged
          (docs/papers/layer-aware-v-compression.md:24-27, docs/benchmarks.md:21-41)
Layers are counted over the layers that own a KV cache (the fix the paper asks
for on hybrid models, layer-aware-v-compression.md:156,185): pass that count.

`LayerKV` turns one layer's pair of formats into the store and attention calls
of this package, so a model loop can hold a list of them.
"""
from __future__ import annotations

from dataclasses import dataclass

from . import _lib as L
from .turbo import DecodeAttention, TurboCodec, packed_bytes, q8_0_append, q8_0_store

FORMATS = ("q8_0", "turbo4", "turbo3", "turbo2")

# bits per value as the fork's tables count them (32-value blocks with an fp16 scale or norm:
# layer-aware-v-compression.md:25-26,51; turbo4 from docs/papers/turbo4-resurrection.md:21)
FORK_BITS = {"q8_0": 8.5, "turbo4": 4.25, "turbo3": 3.5, "turbo2": 2.5}
# bits per value of this package's 128-token blocks (one fp16 norm per 128 values; q8_0 rows keep 4 scales)
BLOCK_BITS = {"q8_0": 8.5, "turbo4": 4.125, "turbo3": 3.125, "turbo2": 2.125}

MODES = (0, 1, 2, 5, 6, 7)


@dataclass(frozen=True)
class LayerFormat:
    k: str
    v: str


def _check_format(name: str) -> str:
    if name not in FORMATS:
        raise ValueError(f"cache format must be one of {FORMATS}, got {name!r}")
    return name


def layer_formats(n_layers: int, mode: int, k: str = "q8_0", v: str = "turbo2") -> list[LayerFormat]:
    """Formats of the n_layers KV-owning layers under a TURBO_LAYER_ADAPTIVE mode; k / v are the base
    formats (-ctk / -ctv).  Boundary sets larger than the model shrink to the model."""
    if n_layers < 1:
        raise ValueError(f"n_layers must be >= 1, got {n_layers}")
    if mode not in MODES:
        raise ValueError(f"mode must be one of {MODES}, got {mode}")
    base = LayerFormat(_check_format(k), _check_format(v))
    first = {1: 4, 5: 2, 7: 2}.get(mode, 0)
    last = {1: 4, 2: 8, 5: 2, 6: 8, 7: 2}.get(mode, 0)
    out = []
    for i in range(n_layers):
        if i < first or i >= n_layers - last:
            if mode in (1, 2):
                out.append(LayerFormat("q8_0", "q8_0"))
            elif mode in (5, 6):
                out.append(LayerFormat(base.k, "turbo4"))
            else:
                out.append(LayerFormat(base.k, "q8_0"))
        else:
            out.append(base)
    return out


def effective_bits(formats: list[LayerFormat], side: str = "v", table: dict = FORK_BITS) -> float:
    """Mean bits per cached value over the layers, for side "k", "v" or "kv"."""
    if side not in ("k", "v", "kv"):
        raise ValueError(f"side must be 'k', 'v' or 'kv', got {side!r}")
    if not formats:
        raise ValueError("no layers")
    tot = 0.0
    for f in formats:
        if side == "k":
            tot += table[f.k]
        elif side == "v":
            tot += table[f.v]
        else:
            tot += 0.5 * (table[f.k] + table[f.v])
    return tot / len(formats)


class LayerKV:
    """One layer's K and V formats bound to this package's kernels.

    store(k, v) -> (k_packed, v_packed) device buffers; attention(...) -> a
    DecodeAttention over such buffers.  Seeds follow kv_cache.py:95 (V = K + 500).
    """

    def __init__(self, fmt: LayerFormat, seed: int = 42):
        self.format = fmt
        self.k_codec = None if _check_format(fmt.k) == "q8_0" else TurboCodec(int(fmt.k[-1]), seed=seed)
        self.v_codec = None if _check_format(fmt.v) == "q8_0" else TurboCodec(int(fmt.v[-1]), seed=seed + 500)

    def store(self, k, v):
        kp = q8_0_store(k, kind="k")[0] if self.k_codec is None else self.k_codec.store(k, kind="k")
        vp = q8_0_store(v, kind="v")[0] if self.v_codec is None else self.v_codec.store(v, kind="v")
        return kp, vp

    def new_cache(self, n_seqs: int, capacity: int):
        """Zeroed (k, v) buffers for `capacity` tokens per sequence, to be filled by append()."""
        tt = L.torch()
        dev = L.require_gpu()

        def nbytes(codec):
            if codec is None:
                return int(L.lib().tq_q8_0_bytes(n_seqs, capacity))
            return packed_bytes(codec.bits, n_seqs, capacity)
        return (tt.zeros(nbytes(self.k_codec), dtype=tt.uint8, device=dev),
                tt.zeros(nbytes(self.v_codec), dtype=tt.uint8, device=dev))

    def append(self, k, v, k_cache, v_cache, pos, capacity: int, overrun=None):
        """The K and V tokens [n_seqs, n_new, 128] of a decode step at positions pos .. pos+n_new-1 (pos: an int, or an
        int64 device tensor with one element read when the launches run; with such a position `overrun`, a zeroed int32
        device tensor with one element, collects the OVERRUN_* bits of launches that refused the position)."""
        if self.k_codec is not None and self.v_codec is not None:
            self.k_codec.append_kv(self.v_codec, k, v, k_cache, v_cache, pos, capacity, overrun=overrun)
            return k_cache, v_cache
        if self.k_codec is None:
            q8_0_append(k, k_cache, pos, capacity, kind="k", overrun=overrun)
        else:
            self.k_codec.append(k, k_cache, pos, capacity, kind="k", overrun=overrun)
        if self.v_codec is None:
            q8_0_append(v, v_cache, pos, capacity, kind="v", overrun=overrun)
        else:
            self.v_codec.append(v, v_cache, pos, capacity, kind="v", overrun=overrun)
        return k_cache, v_cache

    def prefill(self, k, v, k_cache, v_cache, capacity: int):
        """The prompt's K and V [n_seqs, tokens, 128] into caches laid out for `capacity` tokens, from position 0:
        turbo K with turbo V through the fused store (TurboCodec.store_kv(capacity=...), the matrix-core kernels for
        fp16 rows), any other pair through append() at position 0."""
        if self.k_codec is not None and self.v_codec is not None:
            self.k_codec.store_kv(self.v_codec, k, v, out_k=k_cache, out_v=v_cache, capacity=capacity)
            return k_cache, v_cache
        return self.append(k, v, k_cache, v_cache, 0, capacity)

    def attention(self, batch: int, n_q_heads: int, n_kv_heads: int, tokens: int, **kw) -> DecodeAttention:
        return DecodeAttention(self.k_codec, self.v_codec, batch, n_q_heads, n_kv_heads, tokens, **kw)
