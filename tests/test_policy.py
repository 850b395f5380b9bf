"""Layer-adaptive cache policies: the layer sets and effective bit rates against the figures the
reference's documents print (CPU), and every layer of every mode through the kernels (GPU)."""
import numpy as np
import pytest

import turboquant_plus_amd as tqa
from turboquant_plus_amd import policy as P


def test_boundary_v_layer_sets():
    f = P.layer_formats(40, 7, k="q8_0", v="turbo2")
    # docs/papers/layer-aware-v-compression.md:24-27: layers 0, 1, N-2, N-1 keep V as q8_0, K unchanged
    assert [i for i, x in enumerate(f) if x.v == "q8_0"] == [0, 1, 38, 39]
    assert all(x.k == "q8_0" for x in f) and all(x.v == "turbo2" for x in f[2:38])
    f = P.layer_formats(40, 2, k="turbo3", v="turbo3")
    # docs/experiment-layer-adaptive.md:12,20: q8_0 on the last 8 of 40 layers, 32/40 stay turbo3
    assert [i for i, x in enumerate(f) if x == P.LayerFormat("q8_0", "q8_0")] == list(range(32, 40))
    assert sum(x == P.LayerFormat("turbo3", "turbo3") for x in f) == 32
    f = P.layer_formats(40, 1, k="turbo3", v="turbo3")
    assert [i for i, x in enumerate(f) if x.k == "q8_0"] == [0, 1, 2, 3, 36, 37, 38, 39]
    assert P.layer_formats(12, 0, "turbo4", "turbo2") == [P.LayerFormat("turbo4", "turbo2")] * 12
    f = P.layer_formats(28, 5)
    assert [i for i, x in enumerate(f) if x.v == "turbo4"] == [0, 1, 26, 27]
    f = P.layer_formats(28, 6)
    assert [i for i, x in enumerate(f) if x.v == "turbo4"] == list(range(20, 28))
    # a model smaller than the boundary set
    assert all(x.v == "q8_0" for x in P.layer_formats(3, 7))


@pytest.mark.parametrize("n_layers,bits", [(40, 3.10), (28, 3.36), (64, 2.88)])
def test_boundary_v_effective_bits_match_the_published_table(n_layers, bits):
    # docs/papers/layer-aware-v-compression.md:51-56 (phi-4, Qwen2.5-7B, Qwen3.5-27B as counted there)
    got = P.effective_bits(P.layer_formats(n_layers, 7), "v")
    assert round(got, 2) == bits
    # extra V cost against uniform turbo2, layer-aware-v-compression.md:95-100: +24 %, +34 %, +15 %
    extra = {40: 24, 28: 34, 64: 15}[n_layers]
    assert round(100 * (got / 2.5 - 1)) == extra


def test_block_bits_match_the_packed_sizes():
    for name, b in P.BLOCK_BITS.items():
        nbytes = 128 * 136 if name == "q8_0" else tqa.packed_bytes(int(name[-1]), 1, 128)
        assert nbytes * 8 / (128 * 128) == b


def test_bad_arguments():
    with pytest.raises(ValueError):
        P.layer_formats(0, 7)
    with pytest.raises(ValueError):
        P.layer_formats(8, 3)
    with pytest.raises(ValueError):
        P.layer_formats(8, 7, v="q4_0")
    with pytest.raises(ValueError):
        P.effective_bits([], "v")


@pytest.mark.gpu
@pytest.mark.parametrize("mode,k,v", [(7, "q8_0", "turbo2"), (7, "turbo4", "turbo2"), (2, "turbo3", "turbo3"),
                                      (5, "q8_0", "turbo2"), (1, "turbo3", "turbo3"), (7, "turbo3", "turbo3")])
def test_every_layer_of_a_policy_runs_and_matches_the_oracle(mode, k, v):
    from test_gpu_attention import D, assert_close, np_, reference_attention
    B, Hq, Hkv, N = 1, 8, 2, 700
    formats = P.layer_formats(10, mode, k=k, v=v)
    rng = np.random.default_rng(mode)
    seen = {}
    for i, fmt in enumerate(formats):
        if fmt in seen:      # same formats, same kernels: one check per distinct pair
            continue
        seen[fmt] = i
        layer = tqa.LayerKV(fmt, seed=42 + i)
        kx = rng.standard_normal((B * Hkv, N, D)).astype(np.float16)
        vx = rng.standard_normal((B * Hkv, N, D)).astype(np.float16)
        q = rng.standard_normal((B, Hq, D)).astype(np.float16)
        kp, vp = layer.store(kx, vx)
        out = np_(layer.attention(B, Hq, Hkv, N, n_splits=4)(q, kp, vp))
        ref, _, _ = reference_attention(q, layer.k_codec, layer.v_codec, kp, vp, B, Hq, Hkv, N, 1 / np.sqrt(D),
                                        k_q8=kp if layer.k_codec is None else None,
                                        v_q8=vp if layer.v_codec is None else None)
        assert_close(out, ref)
    assert len(seen) >= (1 if mode == 0 else 2)
