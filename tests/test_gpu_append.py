"""GPU tests of the streaming append (tq_append) and of attention over a cache that
grows in a buffer laid out for a fixed capacity.

The reference only names this step ("compress_token", turboquant/kv_cache.py:65-66) and
does not implement it, so the contract checked here is the library's own: whatever the
chunking, the blocks touched by appends covering tokens 0 .. T-1 hold exactly the bytes
that tq_store writes for the first T tokens (same fp32 butterfly arithmetic), and the
codes agree with the oracle like the store's do."""
import numpy as np
import pytest

import tq_oracle as O
import turboquant_plus_amd as tqa
from turboquant_plus_amd import _lib as L
from test_gpu_turbo import check_codes, np_

pytestmark = pytest.mark.gpu
D = 128


def blocks_of(buf, bits, n_seqs, capacity):
    return np_(buf).reshape(n_seqs, -1, O.block_bytes(bits))


@pytest.mark.parametrize("bits", [2, 3, 4])
@pytest.mark.parametrize("kind", ["k", "v"])
def test_append_in_chunks_equals_store(bits, kind):
    tt = L.torch()
    codec = tqa.TurboCodec(bits, seed=7)
    n_seqs, capacity = 3, 512
    x = np.random.default_rng(bits).standard_normal((n_seqs, 300, D)).astype(np.float32)
    x[1, 5] = 0
    cache = tt.zeros(tqa.packed_bytes(bits, n_seqs, capacity), dtype=tt.uint8, device="cuda")
    pos = 0
    for n_new in [1, 1, 62, 64, 5, 130, 37]:
        codec.append(x[:, pos:pos + n_new], cache, pos, capacity, kind=kind)
        pos += n_new
        want = np_(codec.store(x[:, :pos], kind=kind)).reshape(n_seqs, -1, O.block_bytes(bits))
        got = blocks_of(cache, bits, n_seqs, capacity)
        nb = want.shape[1]
        assert np.array_equal(got[:, :nb], want), f"after {pos} tokens"
        assert not got[:, nb:].any()                       # blocks not reached yet are untouched
    assert pos == 300


@pytest.mark.parametrize("dtype", [np.float16, np.float32])
def test_append_codes_match_oracle(dtype):
    tt = L.torch()
    codec = tqa.TurboCodec(3, seed=11)
    n_seqs, capacity, T = 4, 256, 200
    x = np.random.default_rng(0).standard_normal((n_seqs, T, D)).astype(dtype)
    for kind in ("k", "v"):
        cache = tt.zeros(tqa.packed_bytes(3, n_seqs, capacity), dtype=tt.uint8, device="cuda")
        for pos in range(0, T, 50):
            codec.append(x[:, pos:pos + 50], cache, pos, capacity, kind=kind)
        idx, g = codec.unpack_codes(cache, n_seqs, capacity, kind=kind)
        idx, g = np_(idx).reshape(n_seqs, capacity, D)[:, :T], np_(g).reshape(n_seqs, capacity)[:, :T]
        check_codes(codec, x.reshape(-1, D), idx.reshape(-1, D), g.reshape(-1))


def test_append_rejects_overflow_and_accepts_empty():
    tt = L.torch()
    codec = tqa.TurboCodec(3, seed=1)
    cache = tt.zeros(tqa.packed_bytes(3, 2, 128), dtype=tt.uint8, device="cuda")
    with pytest.raises(ValueError):
        codec.append(np.zeros((2, 2, D), dtype=np.float32), cache, 127, 128)
    with pytest.raises(ValueError):
        codec.append(np.zeros((2, 1, D), dtype=np.float32), cache[:100], 0, 128)
    codec.append(np.zeros((2, 0, D), dtype=np.float32), cache, 5, 128)
    assert not np_(cache).any()


def test_decode_attention_over_a_growing_cache():
    """Token-by-token decode: append K and V of the new token, attend over the prefix.  The
    cache stays in a buffer laid out for `capacity` tokens; every step must equal attention over
    a cache stored at exactly that length."""
    tt = L.torch()
    B, Hq, Hkv, capacity = 2, 8, 2, 384
    kc, vc = tqa.TurboCodec(3, seed=42), tqa.TurboCodec(3, seed=542)
    rng = np.random.default_rng(5)
    k = rng.standard_normal((B * Hkv, 200, D)).astype(np.float32)
    v = rng.standard_normal((B * Hkv, 200, D)).astype(np.float32)
    kcache = tt.zeros(tqa.packed_bytes(3, B * Hkv, capacity), dtype=tt.uint8, device="cuda")
    vcache = tt.zeros_like(kcache)
    prefill = 120
    kc.append(k[:, :prefill], kcache, 0, capacity, kind="k")
    vc.append(v[:, :prefill], vcache, 0, capacity, kind="v")
    grow = tqa.DecodeAttention(kc, vc, B, Hq, Hkv, prefill, capacity=capacity, n_splits=2)
    for T in range(prefill + 1, prefill + 12):
        kc.append(k[:, T - 1:T], kcache, T - 1, capacity, kind="k")
        vc.append(v[:, T - 1:T], vcache, T - 1, capacity, kind="v")
        q = rng.standard_normal((B, Hq, D)).astype(np.float16)
        grow.set_tokens(T)
        got = np_(grow(q, kcache, vcache)).copy()
        exact = tqa.DecodeAttention(kc, vc, B, Hq, Hkv, T, n_splits=2)
        want = np_(exact(q, kc.store(k[:, :T], kind="k"), vc.store(v[:, :T], kind="v")))
        assert np.array_equal(got, want), f"context {T}"
    with pytest.raises(ValueError):
        grow.set_tokens(capacity + 1)
