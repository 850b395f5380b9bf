"""CPU-only checks: the C-ABI library loads and exports every symbol that
include/tq.h declares, argument validation works without a GPU, and the
host-side tables / size arithmetic of the package equal the reference's
(golden vectors).  No kernel is launched here."""
import ctypes as C
import os
import re

import numpy as np
import pytest

import turboquant_plus_amd as tqa
from turboquant_plus_amd import _lib as L
from turboquant_plus_amd import codebook, rotation, utils
from turboquant_plus_amd.qjl import QJL, QJL_CONST

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def header_symbols():
    text = open(os.path.join(ROOT, "include", "tq.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(tq_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = L.lib()
    names = header_symbols()
    assert len(names) >= 25
    for n in names:
        assert hasattr(lib, n), f"{n} declared in tq.h but not exported"
    assert sorted(L.PROTOTYPES) == names, "ctypes prototypes out of sync with include/tq.h"
    assert lib.tq_version() >= 100


def test_size_entry_points_need_no_gpu():
    lib = L.lib()
    assert lib.tq_packed_bytes(3, 1, 128) == 6400          # 50 B per 128 values
    assert lib.tq_packed_bytes(4, 1, 128) == 128 * 66      # 64 B codes + fp16 norm
    assert lib.tq_packed_bytes(2, 1, 128) == 128 * 34
    assert lib.tq_packed_bytes(3, 8, 32768) == 8 * 256 * 6400
    assert lib.tq_packed_bytes(3, 2, 130) == 2 * 2 * 6400  # ragged: two blocks per sequence
    assert lib.tq_packed_bytes(5, 1, 128) == -1
    assert lib.tq_q8_0_bytes(1, 128) == 128 * 136
    # the fork's storage blocks: 128 / block_values blocks of 2 + block_values * bits / 8 bytes per vector
    assert [lib.tq_fork_row_bytes(3, bv) for bv in (32, 64, 128)] == [4 * 14, 2 * 26, 50]
    assert [lib.tq_fork_row_bytes(2, bv) for bv in (32, 64, 128)] == [4 * 10, 2 * 18, 34]
    assert lib.tq_fork_row_bytes(4, 128) == 68 == lib.tq_fork_block_bytes(4)
    assert lib.tq_fork_row_bytes(4, 32) == -1 and lib.tq_fork_row_bytes(3, 16) == -1 and lib.tq_fork_row_bytes(5, 128) == -1
    p = L.TQAttnParams(batch=16, n_q_heads=32, n_kv_heads=8, tokens=32768, n_splits=16,
                       k_format=L.KFMT_TURBO, scale=0.088, sparse_v_tau=0.0)
    # one partial (four heads x (128 outputs + maximum + sum)) per workgroup; the 16 splits of a group go to two
    # workgroups of eight wavefronts (128 workgroups of sixteen would leave half of the CUs without one)
    one_per_group = 16 * 8 * 4 * 130 * 4
    assert 2 * one_per_group <= lib.tq_attn_workspace_bytes(C.byref(p)) < 3 * one_per_group
    p.batch = 64                                           # 512 groups: sixteen splits are one workgroup
    assert 4 * one_per_group <= lib.tq_attn_workspace_bytes(C.byref(p)) < 5 * one_per_group
    p.n_q_heads = 16                                       # groups of 2: two of the four head rows per pass idle
    assert 4 * one_per_group <= lib.tq_attn_workspace_bytes(C.byref(p)) < 5 * one_per_group
    p.batch = 16
    p.n_q_heads, p.n_splits = 64, 32                       # groups of 8: eight heads per pass, eight wavefronts per workgroup
    assert 4 * 2 * one_per_group <= lib.tq_attn_workspace_bytes(C.byref(p)) < 4 * 2 * one_per_group + 65536
    p.n_q_heads, p.n_splits, p.head_dim = 32, 32, 256      # heads of 256 dims: two accumulator sets, like eight heads per pass
    assert 4 * 2 * one_per_group <= lib.tq_attn_workspace_bytes(C.byref(p)) < 4 * 2 * one_per_group + 65536
    p.head_dim = 0
    p.n_splits = 16
    p.n_q_heads = 20                                       # not a multiple of the KV head count
    assert lib.tq_attn_workspace_bytes(C.byref(p)) == -1
    assert "multiple of the KV head count" in L.last_error()


def test_argument_errors_map_to_reference_exceptions():
    lib = L.lib()
    rc = lib.tq_fwht(C.c_void_p(8), C.c_void_p(8), 1, 12, L.TQ_F64, L.TQ_F64, None)
    assert rc == L.ERR_ARG
    with pytest.raises(ValueError, match="power of 2"):
        L.check(rc)
    rc = lib.tq_pack_indices(C.c_void_p(8), 4, 9, C.c_void_p(8), None)
    with pytest.raises(ValueError, match="bit_width must be 1-8"):
        L.check(rc)
    assert lib.tq_rotate(None, None, None, 1, 0, 0, 0, None) == L.ERR_ARG
    assert lib.tq_store(None, C.c_void_p(16), 1, 1, 0, 0, C.c_void_p(16), None) == L.ERR_ARG
    h = C.c_void_p()
    assert lib.tq_create(C.byref(h), None) == L.ERR_ARG
    cent = np.array([-1.0, 1.0])
    cfg = L.TQConfig(d=8192, bits=1, rotation=L.ROT_WHT, norm_correction=1, centroids=L.dbl_ptr(cent))
    assert lib.tq_create(C.byref(h), C.byref(cfg)) == L.ERR_UNSUPPORTED


def test_no_gpu_means_loud_failure():
    if L.lib().tq_device_count() > 0:
        pytest.skip("a GPU is visible")
    with pytest.raises(RuntimeError, match="no HIP device"):
        tqa.PolarQuant(128, 3).quantize(np.ones(128))
    with pytest.raises(RuntimeError, match="no HIP device"):
        rotation.fast_walsh_hadamard_transform(np.ones(8))
    with pytest.raises(RuntimeError, match="no HIP device"):
        tqa.TurboCodec(3).store(np.ones((128, 128), dtype=np.float32))


def test_package_does_not_import_the_oracle():
    pkg = os.path.join(ROOT, "turboquant_plus_amd")
    for fn in os.listdir(pkg):
        if fn.endswith(".py"):
            src = open(os.path.join(pkg, fn)).read()
            assert "tq_oracle" not in src and "oracle" not in re.findall(r"^\s*(?:from|import)\s+(\w+)", src, re.M)


# ---- host tables equal the reference's -------------------------------------------

@pytest.mark.parametrize("b", [1, 2, 3, 4])
@pytest.mark.parametrize("d", [64, 128, 256])
def test_optimal_centroids(golden, b, d):
    assert np.array_equal(codebook.optimal_centroids(b, d), golden[f"centroids_b{b}_d{d}"])


def test_conditional_expectation(golden):
    got = np.array([codebook._gaussian_conditional_expectation(*r) for r in golden["cond_mean_args"]])
    assert np.array_equal(got, golden["cond_mean_vals"])


def test_rotation_tables(golden):
    np.testing.assert_allclose(rotation.random_rotation_dense(128, np.random.default_rng(42)), golden["haar_seed42"],
                               rtol=0, atol=1e-13)
    s1, s2, pd = rotation.random_rotation_fast(128, np.random.default_rng(1))
    assert pd == 128 and np.array_equal(s1, golden["fast_s1_seed1"]) and np.array_equal(s2, golden["fast_s2_seed1"])
    s1, s2, pd = rotation.random_rotation_fast(100, np.random.default_rng(9))
    assert pd == 128 and np.array_equal(s1, golden["fast_s1_d100_seed9"])
    assert np.array_equal(rotation.hadamard_matrix(8), golden["hadamard_8"])
    with pytest.raises(ValueError, match="power of 2"):
        rotation.hadamard_matrix(6)
    with pytest.raises(ValueError, match="d must be >= 1"):
        rotation.random_rotation_dense(0, np.random.default_rng(0))
    with pytest.raises(ValueError, match="power of 2"):
        rotation.fast_walsh_hadamard_transform(np.ones(12))


def test_quantiser_tables_and_seeds(golden):
    pq = tqa.PolarQuant(128, 3, seed=42)
    np.testing.assert_allclose(pq.rotation, golden["haar_seed42"], rtol=0, atol=1e-13)
    assert np.array_equal(pq.centroids, golden["centroids_b3_d128"]) and pq.n_centroids == 8
    np.testing.assert_allclose(QJL(128, seed=123).S, golden["qjl_S_seed123"], rtol=0, atol=1e-13)
    tq = tqa.TurboQuant(128, 3, seed=42)
    np.testing.assert_allclose(tq.qjl.S[0], golden["qjl_S_seed1042_row0"], rtol=0, atol=1e-13)  # seed + 1000
    assert tq.polar_quant.bit_width == 2
    kv = tqa.KVCacheCompressor(128, 3, 3, seed=42)
    np.testing.assert_allclose(kv.v_quantizer.polar_quant.rotation, golden["haar_seed542"], rtol=0, atol=1e-13)
    assert abs(QJL_CONST - np.sqrt(np.pi / 2)) < 1e-15
    for d in (64, 128, 256):
        S = QJL(d).S
        assert np.linalg.norm(S @ S.T - np.eye(d), "fro") < 1e-12
    with pytest.raises(ValueError, match="bit_width >= 2"):
        tqa.TurboQuant(128, 1)
    codec = tqa.TurboCodec(3, seed=1, single_diagonal=True)
    assert np.array_equal(codec.signs1, golden["c1_signs"]) and np.all(codec.signs2 == 1)


def test_size_arithmetic(golden):
    for b in (2, 3, 4):
        tq = tqa.TurboQuant(128, b)
        assert tq.compressed_size_bits(100) == int(golden[f"tq_size_bits_b{b}"])
        assert tq.compression_ratio() == float(golden[f"tq_ratio_b{b}"])
    assert tqa.TurboQuant(128, 3).compressed_size_bits(100) == 100 * (128 * 3 + 32)
    ms = tqa.KVCacheCompressor(128, 3, 3).memory_stats(1024, 32, 8)
    got = [ms["original_mb"], ms["compressed_mb"], ms["compression_ratio"], ms["k_bits_per_value"], ms["v_bits_per_value"]]
    assert np.array_equal(np.array(got, dtype=np.float64), golden["kv_memory_stats"])
    fp = utils.memory_footprint_bytes(1000, 128, 3)
    got = [fp["mse_indices_bytes"], fp["qjl_signs_bytes"], fp["norms_bytes"], fp["total_bytes"], fp["original_fp16_bytes"]]
    assert np.array_equal(np.array(got), golden["footprint_1000_128_3"])
    assert fp["mse_indices_bytes"] + fp["qjl_signs_bytes"] + fp["norms_bytes"] == fp["total_bytes"]
    with pytest.raises(ValueError, match="bit_width must be 1-8"):
        utils.pack_indices(np.zeros(4, dtype=np.int64), 9)
    assert utils.pack_indices(np.array([200, 3]), 8).tolist() == [200, 3]


def test_kv_shape_asserts():
    kv = tqa.KVCacheCompressor(64, 3, 3)
    with pytest.raises(AssertionError):
        kv.compress(np.zeros((1, 1, 4, 32)), np.zeros((1, 1, 4, 32)))
    with pytest.raises(AssertionError):
        kv.compress(np.zeros((1, 1, 4, 64)), np.zeros((1, 1, 5, 64)))


def test_requantize_rejects_another_rotation():
    """Codes written under one rotation mean nothing under another: the check is made on the host tables,
    before any device work."""
    a, b = tqa.TurboCodec(3, seed=1), tqa.TurboCodec(2, seed=501)
    with pytest.raises(ValueError, match="same rotation"):
        a.requantize_to(b, None, 1, 128)


def test_probe_library_is_separate_from_the_codec_abi():
    """The benchmark's probes live in their own library and header; the codec's header and library do not
    carry them."""
    from turboquant_plus_amd import probes
    assert not any(n.startswith("tq_probe") for n in header_symbols())
    assert not hasattr(L.lib(), "tq_probe_stream")
    assert all(hasattr(probes.lib(), n) for n in ("tq_probe_stream", "tq_probe_flat", "tq_probe_mfma_f16"))
