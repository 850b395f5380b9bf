"""GPU parity of the reference-API classes (float64 HIP kernels) against the
oracle, the golden vectors written from the reference, and the invariants the
reference's own tests assert (tests/test_rotation.py, test_codebook.py,
test_polar_quant.py, test_qjl.py, test_turboquant.py, test_turbo4.py,
test_kv_cache.py, test_distortion.py, test_utils.py).

Tolerances: codebook indices and sign bits bit-exact; float64 outputs to
1e-12 relative (the GPU sums 128-term dot products in a different order than
BLAS); the float64 WHT uses the reference's stage order and is bit-exact."""
import numpy as np
import pytest
import scipy.linalg

import tq_oracle as O
import turboquant_plus_amd as tqa
from turboquant_plus_amd import codebook, rotation, utils

pytestmark = pytest.mark.gpu
D = 128


def unit(n, d, seed):
    x = np.random.default_rng(seed).standard_normal((n, d))
    return x / np.linalg.norm(x, axis=1, keepdims=True)


# ---- rotation (tests/test_rotation.py) -------------------------------------------

@pytest.mark.parametrize("n", [1, 2, 8, 64, 128, 1024])
def test_fwht_equals_scipy_hadamard_and_oracle(n):
    x = np.random.default_rng(n).standard_normal(n)
    y = rotation.fast_walsh_hadamard_transform(x)
    assert y.dtype == np.float64
    np.testing.assert_allclose(y, scipy.linalg.hadamard(n) @ x / np.sqrt(n), atol=1e-10)
    assert np.array_equal(y, O.fwht(x))          # same stage order -> same bits
    np.testing.assert_allclose(rotation.fast_walsh_hadamard_transform(y), x, atol=1e-10)


def test_fast_rotation_golden(golden):
    s1, s2 = golden["fast_s1_seed1"], golden["fast_s2_seed1"]
    x = golden["rot_x"]
    assert np.array_equal(rotation.fast_walsh_hadamard_transform(x[0]), golden["fwht_x0"])
    assert np.array_equal(rotation.apply_fast_rotation(x[1], s1, s2, 128), golden["rot_single"])
    assert np.array_equal(rotation.apply_fast_rotation_transpose(x[2], s1, s2, 128), golden["rot_single_T"])
    assert np.array_equal(rotation.apply_fast_rotation_batch(x, s1, s2, 128), golden["rot_batch"])
    got = rotation.apply_fast_rotation_batch(golden["rot_x100"], golden["fast_s1_d100_seed9"],
                                             golden["fast_s2_d100_seed9"], 128)
    assert got.shape == (8, 100) and np.array_equal(got, golden["rot_batch_d100"])


@pytest.mark.parametrize("d", [64, 100, 128, 256])
def test_fast_rotation_properties(d):
    rng = np.random.default_rng(d)
    s1, s2, pd = rotation.random_rotation_fast(d, rng)
    x = rng.standard_normal((5, d))
    y = rotation.apply_fast_rotation_batch(x, s1, s2, pd)
    assert y.shape == (5, d)
    for i in range(5):
        np.testing.assert_allclose(rotation.apply_fast_rotation(x[i], s1, s2, pd), y[i], atol=1e-10)
    if d == pd:
        np.testing.assert_allclose(np.linalg.norm(y, axis=1), np.linalg.norm(x, axis=1), rtol=1e-10)
        back = rotation.apply_fast_rotation_transpose(y[0], s1, s2, pd)
        np.testing.assert_allclose(back, x[0], atol=1e-10)


# ---- codebook (tests/test_codebook.py) ----------------------------------------------

@pytest.mark.parametrize("b", [1, 2, 3, 4, 6])
def test_nearest_centroid_is_argmin(golden, b):
    c = codebook.optimal_centroids(b, D)
    v = np.random.default_rng(b).standard_normal((25, 20)) / np.sqrt(D)
    idx = codebook.nearest_centroid_indices(v, c)
    assert idx.shape == v.shape and idx.dtype == np.intp
    assert np.array_equal(idx, np.argmin(np.abs(v[..., None] - c), axis=-1))
    assert codebook.nearest_centroid_indices(np.array([-9.0, 9.0]), c).tolist() == [0, len(c) - 1]
    if b == 3:
        assert np.array_equal(codebook.nearest_centroid_indices(golden["nearest_values"], c), golden["nearest_idx_b3"])


# ---- PolarQuant (tests/test_polar_quant.py, test_distortion.py) -----------------------

@pytest.mark.parametrize("b", [1, 2, 3, 4])
def test_polar_quant_golden(golden, b):
    pq = tqa.PolarQuant(D, b, seed=42)
    x = golden["pq_x"]
    idx, n = pq.quantize(x)
    assert idx.dtype == np.int64 and n.dtype == np.float64
    assert np.array_equal(idx, golden[f"pq_idx_b{b}"])
    np.testing.assert_allclose(n, golden[f"pq_norms_b{b}"], rtol=1e-14)
    xh = pq.dequantize(idx, n)
    np.testing.assert_allclose(xh, golden[f"pq_deq_b{b}"], rtol=1e-12, atol=1e-13)
    assert np.all(xh[5] == 0)                              # zero vector -> exactly zero


def test_polar_quant_variants(golden):
    x = golden["pq_x"]
    pq = tqa.PolarQuant(D, 3, seed=42, norm_correction=False)
    np.testing.assert_allclose(pq.dequantize(*pq.quantize(x)), golden["pq_deq_b3_nocorr"], rtol=1e-12, atol=1e-13)
    idx, n, res = tqa.PolarQuant(D, 2, seed=42).quantize_and_residual(x)
    np.testing.assert_allclose(res, golden["pq_residual_b2"], rtol=1e-11, atol=1e-11)
    np.testing.assert_allclose(res, x - tqa.PolarQuant(D, 2, seed=42).dequantize(idx, n), atol=1e-12)
    i1, n1 = tqa.PolarQuant(D, 3, seed=42).quantize(x[3])
    assert i1.shape == (D,) and np.shape(n1) == ()
    assert np.array_equal(i1, golden["pq_single_idx_b3"]) and abs(n1 - golden["pq_single_norm_b3"]) < 1e-13
    one = tqa.PolarQuant(D, 3, seed=42).dequantize(i1, n1)
    assert one.shape == (D,)
    # float32 / float16 inputs are promoted like NumPy does
    i32, n32 = tqa.PolarQuant(D, 3, seed=42).quantize(x.astype(np.float32))
    io, no = O.PolarRef(D, 3, seed=42).quantize(x.astype(np.float32))
    assert np.array_equal(i32, io) and np.allclose(n32, no, rtol=1e-14)


@pytest.mark.parametrize("d", [64, 96, 128, 160, 256, 320, 512])
@pytest.mark.parametrize("b", [2, 3])
def test_polar_quant_vs_oracle_any_dim(d, b):
    x = np.random.default_rng(d + b).standard_normal((33, d))
    g, o = tqa.PolarQuant(d, b, seed=7), O.PolarRef(d, b, seed=7)
    ig, ng = g.quantize(x)
    io, no = o.quantize(x)
    y, _ = o.rotated(x)
    n_bad, n_inadm = O.boundary_band_mismatches(y, ig, o.centroids, rel=1e-12)
    assert n_inadm == 0 and n_bad <= 2, (n_bad, n_inadm)
    np.testing.assert_allclose(ng, no, rtol=1e-14)
    np.testing.assert_allclose(g.dequantize(io, no), o.dequantize(io, no), rtol=1e-11, atol=1e-13)
    assert not np.isnan(g.dequantize(ig, ng)).any()


@pytest.mark.parametrize("b,bound", [(1, 0.36), (2, 0.117), (3, 0.03), (4, 0.009)])
def test_polar_quant_paper_mse_bound(b, bound):
    x = unit(500, D, b)
    pq = tqa.PolarQuant(D, b, seed=42)
    mse = np.mean(np.sum((pq.dequantize(*pq.quantize(x)) - x) ** 2, axis=1))
    assert mse < 2 * bound


def test_polar_quant_wht_mode_matches_oracle():
    x = np.random.default_rng(3).standard_normal((40, D))
    for d in (D, 100):
        xs = x[:, :d]
        g, o = tqa.PolarQuant(d, 3, seed=5, rotation="wht"), O.PolarRef(d, 3, seed=5, rotation="wht")
        ig, ng = g.quantize(xs)
        io, no = o.quantize(xs)
        assert np.array_equal(ig, io)                      # float64 WHT is bit-identical
        np.testing.assert_allclose(g.dequantize(ig, ng), o.dequantize(io, no), rtol=1e-12, atol=1e-14)


# ---- QJL (tests/test_qjl.py) --------------------------------------------------------------

def test_qjl_golden(golden):
    qj = tqa.QJL(D, seed=123)
    z, n = qj.quantize(golden["pq_x"])
    assert z.dtype == np.int8 and set(np.unique(z)) <= {-1, 1}
    assert np.array_equal(z, golden["qjl_signs"])
    np.testing.assert_allclose(n, golden["qjl_norms"], rtol=1e-14)
    assert n[5] == 0 and np.all(z[5] == 1)                 # zero vector: norm 0, signs +1
    np.testing.assert_allclose(qj.dequantize(z, n), golden["qjl_deq"], rtol=1e-12, atol=1e-13)
    np.testing.assert_allclose(qj.dequantize(z, n, shrinkage=2 / np.pi), golden["qjl_deq_shrunk"], rtol=1e-12, atol=1e-13)
    z1, n1 = qj.quantize(golden["pq_x"][2])
    assert z1.shape == (D,) and np.shape(n1) == () and np.array_equal(z1, z[2])
    np.testing.assert_allclose(qj.dequantize(z1, n1), golden["qjl_deq"][2], rtol=1e-12, atol=1e-13)


@pytest.mark.parametrize("mode", ["orthogonal", "gaussian"])
def test_qjl_modes_vs_oracle(mode):
    x = np.random.default_rng(4).standard_normal((50, D))
    g, o = tqa.QJL(D, seed=2, projection=mode), O.QJLRef(D, seed=2, projection=mode)
    zg, ng = g.quantize(x)
    zo, no = o.quantize(x)
    bad = zg != zo
    assert np.all(np.abs(o.project(x))[bad] <= 1e-12 * np.linalg.norm(x, axis=1).max())
    np.testing.assert_allclose(g.dequantize(zo, no), o.dequantize(zo, no), rtol=1e-11, atol=1e-13)


def test_qjl_single_side_inner_product_unbiased():
    rng = np.random.default_rng(0)
    x, y = rng.standard_normal(D), rng.standard_normal(D)
    est = []
    for s in range(60):
        qj = tqa.QJL(D, seed=s)
        z, n = qj.quantize(x)
        est.append(qj.dequantize(z, n) @ y)
    se = np.std(est) / np.sqrt(len(est))
    assert abs(np.mean(est) - x @ y) < 3 * se + 0.1


# ---- TurboQuant (tests/test_turboquant.py, test_turbo4.py) -------------------------------

@pytest.mark.parametrize("b", [2, 3, 4])
def test_turboquant_golden(golden, b):
    tq = tqa.TurboQuant(D, b, seed=42)
    c = tq.quantize(golden["pq_x"])
    assert c.bit_width == b
    assert np.array_equal(c.mse_indices, golden[f"tq_idx_b{b}"])
    assert np.array_equal(c.qjl_signs, golden[f"tq_signs_b{b}"])
    np.testing.assert_allclose(c.vector_norms, golden[f"tq_vnorm_b{b}"], rtol=1e-14)
    np.testing.assert_allclose(c.residual_norms, golden[f"tq_rnorm_b{b}"], rtol=1e-11, atol=1e-13)
    np.testing.assert_allclose(tq.dequantize(c), golden[f"tq_deq_b{b}"], rtol=1e-11, atol=1e-12)
    np.testing.assert_allclose(tq.dequantize(c, shrinkage=2 / np.pi), golden[f"tq_deq_shrunk_b{b}"], rtol=1e-11, atol=1e-12)
    single = tq.quantize(golden["pq_x"][1])
    assert single.mse_indices.shape == (D,) and np.shape(single.vector_norms) == () and np.shape(single.residual_norms) == ()
    np.testing.assert_allclose(tq.dequantize(single), golden[f"tq_deq_b{b}"][1], rtol=1e-10, atol=1e-12)


@pytest.mark.parametrize("tb", [2.5, 3.5])
def test_outlier_turboquant_golden(golden, tb):
    """OutlierTurboQuant (turboquant/outlier.py:70-217) against vectors written from the reference; the
    properties are those of the reference's tests/test_outlier.py."""
    tag = f"outlier_{str(tb).replace('.', 'p')}"
    oq = tqa.OutlierTurboQuant(D, tb, seed=42)
    meta = golden[f"{tag}_meta"]
    assert [oq.n_outlier, oq.high_bits, oq.n_normal, oq.low_bits] == [int(v) for v in meta[:4]]
    assert oq.effective_bits == pytest.approx(tb, abs=0.01)
    assert oq.compression_ratio() == meta[5] and oq.compression_ratio(32) == meta[6]
    x = golden["outlier_x"]
    c = oq.quantize(x)
    assert c.effective_bits == oq.effective_bits
    assert np.array_equal(c.outlier_indices, golden[f"{tag}_oidx"]) and np.array_equal(c.normal_indices, golden[f"{tag}_nidx"])
    assert np.array_equal(c.qjl_signs, golden[f"{tag}_signs"])
    np.testing.assert_allclose(c.outlier_norms, golden[f"{tag}_onorm"], rtol=1e-14)
    np.testing.assert_allclose(c.normal_norms, golden[f"{tag}_nnorm"], rtol=1e-14)
    np.testing.assert_allclose(c.residual_norms, golden[f"{tag}_rnorm"], rtol=1e-11, atol=1e-13)
    deq = oq.dequantize(c)
    np.testing.assert_allclose(deq, golden[f"{tag}_deq"], rtol=1e-11, atol=1e-12)
    # batch == single, determinism (tests/test_outlier.py:81-112)
    for i in (0, 1, 4):
        np.testing.assert_allclose(oq.dequantize(oq.quantize(x[i])), deq[i], atol=1e-10)
    np.testing.assert_allclose(oq.dequantize(oq.quantize(x[1])), golden[f"{tag}_single_deq"], rtol=1e-11, atol=1e-12)
    assert np.array_equal(tqa.OutlierTurboQuant(D, tb, seed=42).dequantize(c), deq)


def test_outlier_turboquant_quality_and_whole_bits():
    rng = np.random.default_rng(3)
    x = rng.standard_normal((200, D))
    x /= np.linalg.norm(x, axis=1, keepdims=True)
    oq = tqa.OutlierTurboQuant(D, 3.5, seed=42)
    mse = np.mean(np.sum((oq.dequantize(oq.quantize(x)) - x) ** 2, axis=1))
    assert mse < 0.03 * 2.0                                  # tests/test_outlier.py:30-48
    whole = tqa.OutlierTurboQuant(D, 3.0, seed=42)           # no high-rate channels
    assert whole.pq_outlier is None and whole.n_normal == D
    assert whole.dequantize(whole.quantize(x[:3])).shape == (3, D)
    assert tqa.OutlierTurboQuant(D, 2.5).compression_ratio() > 4.5 and tqa.OutlierTurboQuant(D, 3.5).compression_ratio() > 3.5


@pytest.mark.parametrize("d", [96, 160, 192, 320])
def test_turbo4_non_power_of_two_dims(d):
    x = np.random.default_rng(d).standard_normal((20, d))
    g, o = tqa.TurboQuant(d, 4, seed=42), O.TurboRef(d, 4, seed=42)
    xg, xo = g.dequantize(g.quantize(x)), o.dequantize(o.quantize(x))
    assert not np.isnan(xg).any()
    np.testing.assert_allclose(xg, xo, rtol=1e-9, atol=1e-10)


def test_turboquant_properties():
    x = unit(200, D, 9)
    mses = {}
    for b, bound in ((2, 0.117), (3, 0.03), (4, 0.009)):
        tq = tqa.TurboQuant(D, b, seed=42)
        xh = tq.dequantize(tq.quantize(x))
        mses[b] = np.mean(np.sum((xh - x) ** 2, axis=1))
    assert mses[2] < 3 * 0.36 and mses[4] < mses[3] < mses[2]
    mse = tqa.TurboQuantMSE(D, 3, seed=42)
    i, n = mse.quantize(x)
    assert np.mean(np.sum((mse.dequantize(i, n) - x) ** 2, axis=1)) < 0.1
    z = tqa.TurboQuant(D, 4).dequantize(tqa.TurboQuant(D, 4).quantize(np.zeros(D)))
    assert np.linalg.norm(z) <= 1e-6
    for scale in (1e-3, 1.0, 1e4):
        tq = tqa.TurboQuant(D, 4, seed=42)
        xs = x[:10] * scale
        err = np.linalg.norm(tq.dequantize(tq.quantize(xs)) - xs, axis=1) / np.linalg.norm(xs, axis=1)
        assert err.max() < 0.6


# ---- KV cache (tests/test_kv_cache.py) ----------------------------------------------------

def test_kv_cache_golden(golden):
    kv = tqa.KVCacheCompressor(D, 3, 3, seed=42)
    c = kv.compress(golden["kv_k"], golden["kv_v"])
    assert (c.num_layers, c.num_heads, c.seq_len, c.head_dim, c.k_bit_width, c.v_bit_width) == (1, 2, 16, 128, 3, 3)
    assert np.array_equal(c.k_compressed[0][1].mse_indices, golden["kv_k_idx_l0h1"])
    assert np.array_equal(c.k_compressed[0][1].qjl_signs, golden["kv_k_signs_l0h1"])
    assert np.array_equal(c.v_indices[0][1], golden["kv_v_idx_l0h1"])
    np.testing.assert_allclose(c.v_norms[0][1], golden["kv_v_norms_l0h1"], rtol=1e-14)
    k, v = kv.decompress(c)
    assert k.shape == v.shape == (1, 2, 16, 128)
    np.testing.assert_allclose(k, golden["kv_k_hat"], rtol=1e-10, atol=1e-11)
    np.testing.assert_allclose(v, golden["kv_v_hat"], rtol=1e-10, atol=1e-11)


def test_kv_cache_attention_quality():
    rng = np.random.default_rng(1)
    d, S = 64, 16
    k, v = rng.standard_normal((1, 1, S, d)), rng.standard_normal((1, 1, S, d))
    q = rng.standard_normal((1, d))
    kv = tqa.KVCacheCompressor(d, 3, 3, seed=42)
    kh, vh = kv.decompress(kv.compress(k, v))
    ref = O.softmax_rows(q @ k[0, 0].T / np.sqrt(d)) @ v[0, 0]
    got = O.softmax_rows(q @ kh[0, 0].T / np.sqrt(d)) @ vh[0, 0]
    cos = (ref @ got.T).item() / (np.linalg.norm(ref) * np.linalg.norm(got))
    assert cos > 0.5
    assert kv.memory_stats(1024, 32, 8)["compression_ratio"] > 2


# ---- packing (tests/test_utils.py) -----------------------------------------------------------

def test_pack_helpers(golden):
    assert np.array_equal(utils.pack_bits(golden["pack_signs_in"]), golden["pack_signs_out"])
    assert np.array_equal(utils.pack_bits(golden["pack_signs_in"][0, :5]), golden["pack_signs_d5_out"])
    assert np.array_equal(utils.unpack_bits(golden["pack_signs_out"], 128), golden["pack_signs_in"])
    assert np.array_equal(utils.unpack_bits(golden["pack_signs_d5_out"], 5), golden["pack_signs_in"][0, :5])
    assert utils.pack_bits(np.ones(128, dtype=np.int8)).shape == (16,)
    assert utils.pack_bits(np.array([1, -1, 1, 1, -1, -1, 1, -1], dtype=np.int8)).tolist() == [0b10110010]
    for b in (1, 2, 3, 4):
        assert np.array_equal(utils.pack_indices(golden[f"pack_idx_in_b{b}"], b), golden[f"pack_idx_out_b{b}"])
    assert utils.pack_indices(np.array([3, 0, 1, 2]), 2).tolist() == [0b11000110]


# ---- wide vectors (PLAN.md:104-108,146: d = 1536 and 3072) -----------------------------------------

@pytest.mark.parametrize("d", [1536, 3072])
def test_wide_dims_match_the_oracle(d):
    """PolarQuant, QJL and TurboQuant at the embedding widths the reference plans to test (1536, 3072): indices
    and sign bits against the oracle built from the same seeds, float64 outputs to 1e-10 (d-term sums in another
    order than BLAS), with the dense Haar rotation and in WHT mode (1536 and 3072 are padded to 2048 and 4096)."""
    rng = np.random.default_rng(d)
    x = rng.standard_normal((5, d))
    x[3] = 0.0
    for rot in ("dense", "wht"):
        g, o = tqa.PolarQuant(d, 3, seed=11, rotation=rot), O.PolarRef(d, 3, seed=11, rotation=rot)
        if rot == "dense":
            assert np.array_equal(g.rotation, o.rotation)
        ig, ng = g.quantize(x)
        io, no = o.quantize(x)
        y, _ = o.rotated(x)
        n_bad, n_inadm = O.boundary_band_mismatches(y, ig, o.centroids, rel=1e-11)
        assert n_inadm == 0 and n_bad <= 2, (rot, n_bad, n_inadm)
        np.testing.assert_allclose(ng, no, rtol=1e-13)
        np.testing.assert_allclose(g.dequantize(io, no), o.dequantize(io, no), rtol=1e-9, atol=1e-12)
        assert np.all(g.dequantize(ig, ng)[3] == 0)
    qg, qo = tqa.QJL(d, seed=5), O.QJLRef(d, seed=5)
    r = rng.standard_normal((4, d))
    sg, ng = qg.quantize(r)
    so, no = qo.quantize(r)
    proj = qo.project(r)
    differ = sg != so
    assert np.all(np.abs(proj[differ]) <= 1e-11 * np.linalg.norm(r, axis=1).max())      # sign flips only at |S r| ~ 0
    assert differ.sum() <= 2
    np.testing.assert_allclose(qg.dequantize(so, no), qo.dequantize(so, no), rtol=1e-9, atol=1e-12)
    if d == 1536:
        tg, to = tqa.TurboQuant(d, 3, seed=42), O.TurboRef(d, 3, seed=42)
        xg, xo = tg.dequantize(tg.quantize(x)), to.dequantize(to.quantize(x))
        np.testing.assert_allclose(xg, xo, rtol=1e-8, atol=1e-10)
        assert tg.compressed_size_bits(7) == 7 * (d * 3 + 32)


@pytest.mark.parametrize("n", [2048, 4096])
def test_fwht_wide(n):
    x = np.random.default_rng(n).standard_normal((3, n))
    got = rotation.fast_walsh_hadamard_transform(x[0])
    assert np.array_equal(got, O.fwht(x[0]))
    np.testing.assert_allclose(got, scipy.linalg.hadamard(n) @ x[0] / np.sqrt(n), atol=1e-11)


def test_dims_beyond_the_limit_are_refused():
    with pytest.raises(NotImplementedError, match="1..4096"):
        tqa.PolarQuant(4097, 2, seed=1, rotation="wht").quantize(np.zeros(4097))


# ---- inner-product distortion (tests/test_distortion.py:78-108,138-157) -----------------------------------

@pytest.mark.parametrize("b", [2, 3, 4])
def test_inner_product_distortion_single_side(b):
    """Paper Theorem 2: E|<y,x> - <y, Q^-1(Q(x))>|^2 <= sqrt(3 pi^2) |y|^2 / d / 4^b with only x quantised;
    1000 unit pairs at d = 256, five times the bound allowed for finite d, as the reference's test does."""
    d = 256
    rng = np.random.default_rng(456)
    x, y = rng.standard_normal((1000, d)), rng.standard_normal((1000, d))
    x /= np.linalg.norm(x, axis=1, keepdims=True)
    y /= np.linalg.norm(y, axis=1, keepdims=True)
    tq = tqa.TurboQuant(d, b, seed=42)
    x_hat = tq.dequantize(tq.quantize(x))
    sq = (np.sum(y * x, axis=1) - np.sum(y * x_hat, axis=1)) ** 2
    bound = np.sqrt(3 * np.pi ** 2) / d / 4 ** b
    assert sq.mean() < 5.0 * bound, (sq.mean(), bound)
    # the estimate is unbiased over pairs: the mean error is within four standard errors of zero
    err = np.sum(y * x_hat, axis=1) - np.sum(y * x, axis=1)
    assert abs(err.mean()) < 4 * err.std() / np.sqrt(err.size)


def test_inner_product_error_decreases_with_bits():
    d = 256
    rng = np.random.default_rng(456)
    x, y = rng.standard_normal((200, d)), rng.standard_normal((200, d))
    x /= np.linalg.norm(x, axis=1, keepdims=True)
    y /= np.linalg.norm(y, axis=1, keepdims=True)
    errs = {}
    for b in (2, 3, 4):
        tq = tqa.TurboQuant(d, b, seed=42)
        errs[b] = np.abs(np.sum(y * x, axis=1) - np.sum(y * tq.dequantize(tq.quantize(x)), axis=1)).mean()
    assert errs[2] > errs[3] > errs[4], errs


def test_mse_decreases_with_bits_and_both_sides_quantised():
    """tests/test_distortion.py:163-178 (monotone MSE at d = 256) and :181-207 (both vectors quantised: TurboQuant's
    inner products stay finite and of the size of PolarQuant's; the reference only prints the two numbers)."""
    d = 256
    rng = np.random.default_rng(789)
    X = rng.standard_normal((200, d))
    X /= np.linalg.norm(X, axis=1, keepdims=True)
    mses = {}
    for b in (1, 2, 3):
        pq = tqa.PolarQuant(d, b, seed=42)
        mses[b] = np.mean((pq.dequantize(*pq.quantize(X)) - X) ** 2)
    assert mses[1] > mses[2] > mses[3]
    Y = rng.standard_normal((200, d))
    Y /= np.linalg.norm(Y, axis=1, keepdims=True)
    pq, tq = tqa.PolarQuant(d, 2, seed=42), tqa.TurboQuant(d, 2, seed=42)
    ip = np.sum(X * Y, axis=1)
    e_pq = np.abs(ip - np.sum(pq.dequantize(*pq.quantize(X)) * pq.dequantize(*pq.quantize(Y)), axis=1)).mean()
    e_tq = np.abs(ip - np.sum(tq.dequantize(tq.quantize(X)) * tq.dequantize(tq.quantize(Y)), axis=1)).mean()
    assert np.isfinite(e_tq) and e_tq < 10 * e_pq
