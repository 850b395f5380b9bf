"""The oracle against vectors written from the reference (tests/golden/)."""
import numpy as np
import pytest

import tq_oracle as O

D = 128


@pytest.mark.parametrize("b", [1, 2, 3, 4])
@pytest.mark.parametrize("d", [64, 128, 256])
def test_centroids_exact(golden, b, d):
    assert np.array_equal(O.centroids_for(b, d), golden[f"centroids_b{b}_d{d}"])


def test_centroids_5bit(golden):
    assert np.array_equal(O.centroids_for(5, 128), golden["centroids_b5_d128"])


def test_conditional_means(golden):
    got = np.array([O.gauss_cond_mean(*r) for r in golden["cond_mean_args"]])
    assert np.array_equal(got, golden["cond_mean_vals"])


def test_nearest_index_including_ties(golden):
    got = O.nearest_index(golden["nearest_values"], golden["centroids_b3_d128"])
    assert np.array_equal(got, golden["nearest_idx_b3"])


@pytest.mark.parametrize("seed", [42, 542])
def test_haar_rotation(golden, seed):
    got = O.haar_rotation(D, np.random.default_rng(seed))
    # same NumPy / LAPACK build -> same bits; a different LAPACK may differ in
    # the last ulps, so the hard assertion is a tight tolerance
    np.testing.assert_allclose(got, golden[f"haar_seed{seed}"], rtol=0, atol=1e-13)


def test_haar_small_and_hadamard(golden):
    np.testing.assert_allclose(O.haar_rotation(16, np.random.default_rng(3)), golden["haar_d16_seed3"], atol=1e-14)
    assert np.array_equal(O.sylvester_hadamard(8), golden["hadamard_8"])


def test_sign_diagonals(golden):
    s1, s2, pd = O.sign_diagonals(D, np.random.default_rng(1))
    assert pd == 128
    assert np.array_equal(s1, golden["fast_s1_seed1"]) and np.array_equal(s2, golden["fast_s2_seed1"])
    s1, s2, pd = O.sign_diagonals(100, np.random.default_rng(9))
    assert pd == 128
    assert np.array_equal(s1, golden["fast_s1_d100_seed9"]) and np.array_equal(s2, golden["fast_s2_d100_seed9"])


def test_fast_rotation(golden):
    x = golden["rot_x"]
    s1, s2 = golden["fast_s1_seed1"], golden["fast_s2_seed1"]
    assert np.array_equal(O.fwht(x[0]), golden["fwht_x0"])
    assert np.array_equal(O.rotate_fast(x[1], s1, s2, 128), golden["rot_single"])
    assert np.array_equal(O.rotate_fast(x[2], s1, s2, 128, transpose=True), golden["rot_single_T"])
    assert np.array_equal(O.rotate_fast(x, s1, s2, 128), golden["rot_batch"])
    got = O.rotate_fast(golden["rot_x100"], golden["fast_s1_d100_seed9"], golden["fast_s2_d100_seed9"], 128)
    assert np.array_equal(got, golden["rot_batch_d100"])


@pytest.mark.parametrize("b", [1, 2, 3, 4])
def test_polar_quant(golden, b):
    pq = O.PolarRef(D, b, seed=42)
    idx, n = pq.quantize(golden["pq_x"])
    assert np.array_equal(idx, golden[f"pq_idx_b{b}"])
    assert np.array_equal(n, golden[f"pq_norms_b{b}"])
    np.testing.assert_allclose(pq.dequantize(idx, n), golden[f"pq_deq_b{b}"], rtol=0, atol=1e-12 * 1e4)
    # the 1e4-scaled row dominates the absolute bound; the others to 1e-13
    rows = [r for r in range(32) if r != 7]
    np.testing.assert_allclose(pq.dequantize(idx, n)[rows], golden[f"pq_deq_b{b}"][rows], rtol=0, atol=1e-13)


def test_polar_quant_variants(golden):
    x = golden["pq_x"]
    pq = O.PolarRef(D, 3, seed=42, norm_correction=False)
    np.testing.assert_allclose(pq.dequantize(*pq.quantize(x)), golden["pq_deq_b3_nocorr"], rtol=1e-12, atol=1e-13)
    _, _, res = O.PolarRef(D, 2, seed=42).quantize_and_residual(x)
    np.testing.assert_allclose(res, golden["pq_residual_b2"], rtol=1e-12, atol=1e-11)
    i1, n1 = O.PolarRef(D, 3, seed=42).quantize(x[3])
    assert np.array_equal(i1, golden["pq_single_idx_b3"]) and n1 == golden["pq_single_norm_b3"]
    assert np.shape(n1) == ()


def test_qjl(golden):
    qj = O.QJLRef(D, seed=123)
    np.testing.assert_allclose(qj.S, golden["qjl_S_seed123"], rtol=0, atol=1e-13)
    z, n = qj.quantize(golden["pq_x"])
    assert z.dtype == np.int8 and np.array_equal(z, golden["qjl_signs"])
    assert np.array_equal(n, golden["qjl_norms"])
    np.testing.assert_allclose(qj.dequantize(z, n), golden["qjl_deq"], rtol=1e-12, atol=1e-13)
    np.testing.assert_allclose(qj.dequantize(z, n, shrinkage=2 / np.pi), golden["qjl_deq_shrunk"], rtol=1e-12, atol=1e-13)
    np.testing.assert_allclose(O.QJLRef(D, seed=1042).S[0], golden["qjl_S_seed1042_row0"], atol=1e-13)


@pytest.mark.parametrize("b", [2, 3, 4])
def test_turboquant(golden, b):
    tq = O.TurboRef(D, b, seed=42)
    c = tq.quantize(golden["pq_x"])
    assert np.array_equal(c.mse_indices, golden[f"tq_idx_b{b}"])
    assert np.array_equal(c.vector_norms, golden[f"tq_vnorm_b{b}"])
    assert np.array_equal(c.qjl_signs, golden[f"tq_signs_b{b}"])
    np.testing.assert_allclose(c.residual_norms, golden[f"tq_rnorm_b{b}"], rtol=1e-12, atol=1e-14)
    np.testing.assert_allclose(tq.dequantize(c), golden[f"tq_deq_b{b}"], rtol=1e-11, atol=1e-12)
    np.testing.assert_allclose(tq.dequantize(c, shrinkage=2 / np.pi), golden[f"tq_deq_shrunk_b{b}"], rtol=1e-11, atol=1e-12)
    assert tq.compressed_size_bits(100) == int(golden[f"tq_size_bits_b{b}"])
    assert tq.compression_ratio() == float(golden[f"tq_ratio_b{b}"])


@pytest.mark.parametrize("tb", [2.5, 3.5])
def test_outlier_split_quantiser(golden, tb):
    """turboquant/outlier.py:45-217 : fractional bit rates by channel split; fixtures written from the reference."""
    tag = f"outlier_{str(tb).replace('.', 'p')}"
    oq = O.OutlierRef(D, tb, seed=42)
    meta = golden[f"{tag}_meta"]
    assert [oq.n_outlier, oq.high_bits, oq.n_normal, oq.low_bits] == [int(v) for v in meta[:4]]
    assert oq.effective_bits == meta[4] and oq.compression_ratio() == meta[5] and oq.compression_ratio(32) == meta[6]
    c = oq.quantize(golden["outlier_x"])
    assert np.array_equal(c[0], golden[f"{tag}_oidx"]) and np.array_equal(c[2], golden[f"{tag}_nidx"])
    assert np.array_equal(c[1], golden[f"{tag}_onorm"]) and np.array_equal(c[3], golden[f"{tag}_nnorm"])
    assert np.array_equal(c[4], golden[f"{tag}_signs"])
    np.testing.assert_allclose(c[5], golden[f"{tag}_rnorm"], rtol=1e-12, atol=1e-14)
    np.testing.assert_allclose(oq.dequantize(c), golden[f"{tag}_deq"], rtol=1e-11, atol=1e-12)
    single = oq.quantize(golden["outlier_x"][1])
    np.testing.assert_allclose(oq.dequantize(single), golden[f"{tag}_single_deq"], rtol=1e-11, atol=1e-12)


def test_outlier_channel_split(golden):
    for (d, tb), want in zip(golden["outlier_split_args"], golden["outlier_split_vals"]):
        assert list(O.channel_split(int(d), float(tb))) == [int(v) for v in want]
    # a whole number of bits leaves no high-rate channels (one PolarQuant only)
    oq = O.OutlierRef(D, 3.0, seed=42)
    assert oq.pq_outlier is None and oq.n_normal == D
    x = np.random.default_rng(0).standard_normal((4, D))
    assert oq.dequantize(oq.quantize(x)).shape == (4, D)


def test_temporal_decay_requantize(golden):
    """3-bit rows -> 2-bit (benchmarks/temporal_decay_prototype.py:93-125); the prototype
    takes the uncorrected norm and corrects at read time, the device format stores the corrected norm."""
    c3, c2 = golden["decay_c3"], golden["decay_c2"]
    idx3, n3 = golden["decay_idx3"], golden["decay_norm3"]
    rn = np.sqrt(np.sum(c3[idx3] ** 2, axis=1))
    g3 = n3 / rn                                        # corrected norm, as dequantize_3bit forms it
    np.testing.assert_allclose(c3[idx3] * g3[:, None], golden["decay_deq3"], rtol=1e-15, atol=0)
    idx2, g2 = O.requantize(idx3, g3, c3, c2, mid_dst=golden["decay_mid2"])
    assert np.array_equal(idx2, golden["decay_idx2"])
    np.testing.assert_allclose(g2, golden["decay_norm2"], rtol=1e-14, atol=0)
    assert g2[5] == 0.0 and np.all(idx2[5] == 2)        # zero row: digitize(0.0) over (-m, 0, m)
    # default midpoints are those of the preset centroids
    np.testing.assert_allclose(O.midpoints(c2), golden["decay_mid2"], atol=1e-12)


def test_kv_cache(golden):
    kv = O.KVRef(D, 3, 3, seed=42)
    c = kv.compress(golden["kv_k"], golden["kv_v"])
    assert np.array_equal(c.k_compressed[0][1].mse_indices, golden["kv_k_idx_l0h1"])
    assert np.array_equal(c.k_compressed[0][1].qjl_signs, golden["kv_k_signs_l0h1"])
    assert np.array_equal(c.v_indices[0][1], golden["kv_v_idx_l0h1"])
    assert np.array_equal(c.v_norms[0][1], golden["kv_v_norms_l0h1"])
    k, v = kv.decompress(c)
    np.testing.assert_allclose(k, golden["kv_k_hat"], rtol=1e-11, atol=1e-12)
    np.testing.assert_allclose(v, golden["kv_v_hat"], rtol=1e-11, atol=1e-12)
    ms = kv.memory_stats(1024, 32, 8)
    got = [ms["original_mb"], ms["compressed_mb"], ms["compression_ratio"], ms["k_bits_per_value"], ms["v_bits_per_value"]]
    assert np.array_equal(np.array(got, dtype=np.float64), golden["kv_memory_stats"])


def test_host_packing(golden):
    assert np.array_equal(O.pack_sign_bits(golden["pack_signs_in"]), golden["pack_signs_out"])
    assert np.array_equal(O.pack_sign_bits(golden["pack_signs_in"][0, :5]), golden["pack_signs_d5_out"])
    assert np.array_equal(O.unpack_sign_bits(golden["pack_signs_out"], 128), golden["pack_signs_in"])
    for b in (1, 2, 3, 4):
        assert np.array_equal(O.pack_index_stream(golden[f"pack_idx_in_b{b}"], b), golden[f"pack_idx_out_b{b}"])
    fp = O.footprint(1000, 128, 3)
    got = [fp["mse_indices_bytes"], fp["qjl_signs_bytes"], fp["norms_bytes"], fp["total_bytes"], fp["original_fp16_bytes"]]
    assert np.array_equal(np.array(got), golden["footprint_1000_128_3"])


def test_config1_composition(golden):
    """BASELINE config 1: seed-0 fp32 data, one seed-1 sign diagonal, WHT,
    8-level codebook; the oracle's production-format encoder must agree with
    the composition of reference functions the fixture was written from."""
    X = np.random.default_rng(0).standard_normal((4096, D)).astype(np.float32)
    s1 = np.random.default_rng(1).choice([-1.0, 1.0], size=D)
    assert np.array_equal(s1, golden["c1_signs"])
    cent = O.centroids_for(3, D)
    idx, g, y = O.turbo_encode(X, s1, np.ones(D), cent, norm_dtype=np.float64)
    assert np.array_equal(idx[:64], golden["c1_idx_first64"])
    assert np.array_equal(np.bincount(idx.ravel(), minlength=8), golden["c1_idx_hist"])
    assert np.array_equal(idx.astype(np.int64).sum(axis=1), golden["c1_idx_rowsum"])
    xh = O.turbo_decode(idx[:64], g[:64], cent, s1, np.ones(D))
    np.testing.assert_allclose(xh, golden["c1_deq_first64"], rtol=1e-12, atol=1e-13)
    rot = O.turbo_decode_rotated(idx, g, cent)
    mse = np.mean((rot - y * golden["c1_norms"][:, None]) ** 2)
    np.testing.assert_allclose(mse, float(golden["c1_mse"]), rtol=1e-10)
