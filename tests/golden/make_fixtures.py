"""Writes tests/golden/reference_vectors.npz from the reference implementation.

Run once, in the build container only (the reference tree does not exist on
the GPU box):

    python tests/golden/make_fixtures.py [/root/reference]

The reference's own tests hold no stored arrays for this path (every numeric
assertion there is a bound or an invariant), so bit-exact agreement with the
reference on seeded inputs can only be shown with vectors written from it.
The file holds inputs and outputs only.
"""
import os
import sys

import numpy as np

ref_root = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
sys.path.insert(0, ref_root)

from turboquant import PolarQuant, QJL, TurboQuant, KVCacheCompressor  # noqa: E402
from turboquant import codebook, rotation, utils  # noqa: E402

out = {}
D = 128

# ---- codebook -------------------------------------------------------------
for b in (1, 2, 3, 4):
    for d in (64, 128, 256):
        out[f"centroids_b{b}_d{d}"] = codebook.optimal_centroids(b, d)
out["centroids_b5_d128"] = codebook.optimal_centroids(5, 128)
out["cond_mean_args"] = np.array([[1.0, -np.inf, 0.0], [1.0, 0.0, np.inf], [0.5, -0.3, 0.7],
                                  [1.0, 40.0, np.inf], [1.0, -np.inf, -40.0], [1.0, 40.0, 40.5]])
out["cond_mean_vals"] = np.array([codebook._gaussian_conditional_expectation(*r) for r in out["cond_mean_args"]])
c3 = out["centroids_b3_d128"]
mid = (c3[:-1] + c3[1:]) / 2
vals = np.concatenate([np.random.default_rng(7).standard_normal(200) / np.sqrt(D), mid, c3, [-1.0, 1.0, 0.0]])
out["nearest_values"] = vals
out["nearest_idx_b3"] = codebook.nearest_centroid_indices(vals, c3)

# ---- rotation -------------------------------------------------------------
for seed in (42, 542):
    out[f"haar_seed{seed}"] = rotation.random_rotation_dense(D, np.random.default_rng(seed))
out["haar_d16_seed3"] = rotation.random_rotation_dense(16, np.random.default_rng(3))
out["hadamard_8"] = rotation.hadamard_matrix(8)
s1, s2, pd = rotation.random_rotation_fast(D, np.random.default_rng(1))
out["fast_s1_seed1"], out["fast_s2_seed1"] = s1, s2
s1b, s2b, pdb = rotation.random_rotation_fast(100, np.random.default_rng(9))
out["fast_s1_d100_seed9"], out["fast_s2_d100_seed9"] = s1b, s2b
xr = np.random.default_rng(11).standard_normal((64, D))
out["rot_x"] = xr
out["fwht_x0"] = rotation.fast_walsh_hadamard_transform(xr[0])
out["rot_single"] = rotation.apply_fast_rotation(xr[1], s1, s2, pd)
out["rot_single_T"] = rotation.apply_fast_rotation_transpose(xr[2], s1, s2, pd)
out["rot_batch"] = rotation.apply_fast_rotation_batch(xr, s1, s2, pd)
x100 = np.random.default_rng(12).standard_normal((8, 100))
out["rot_x100"] = x100
out["rot_batch_d100"] = rotation.apply_fast_rotation_batch(x100, s1b, s2b, pdb)

# ---- quantisers -----------------------------------------------------------
xq = np.random.default_rng(21).standard_normal((32, D))
xq[5] = 0.0
xq[6] *= 1e-3
xq[7] *= 1e4
xq[8, :4] *= 15.0
out["pq_x"] = xq
for b in (1, 2, 3, 4):
    pq = PolarQuant(D, b, seed=42)
    idx, n = pq.quantize(xq)
    out[f"pq_idx_b{b}"] = idx.astype(np.uint8)
    out[f"pq_norms_b{b}"] = n
    out[f"pq_deq_b{b}"] = pq.dequantize(idx, n)
pq = PolarQuant(D, 3, seed=42, norm_correction=False)
idx, n = pq.quantize(xq)
out["pq_deq_b3_nocorr"] = pq.dequantize(idx, n)
idx, n, res = PolarQuant(D, 2, seed=42).quantize_and_residual(xq)
out["pq_residual_b2"] = res
i1, n1 = PolarQuant(D, 3, seed=42).quantize(xq[3])
out["pq_single_idx_b3"] = i1.astype(np.uint8)
out["pq_single_norm_b3"] = np.asarray(n1)

qj = QJL(D, seed=123)
out["qjl_S_seed123"] = qj.S
z, rn = qj.quantize(xq)
out["qjl_signs"], out["qjl_norms"] = z, rn
out["qjl_deq"] = qj.dequantize(z, rn)
out["qjl_deq_shrunk"] = qj.dequantize(z, rn, shrinkage=2 / np.pi)
out["qjl_S_seed1042_row0"] = QJL(D, seed=1042).S[0]

for b in (2, 3, 4):
    tq = TurboQuant(D, b, seed=42)
    c = tq.quantize(xq)
    out[f"tq_idx_b{b}"] = c.mse_indices.astype(np.uint8)
    out[f"tq_vnorm_b{b}"] = c.vector_norms
    out[f"tq_signs_b{b}"] = c.qjl_signs
    out[f"tq_rnorm_b{b}"] = c.residual_norms
    out[f"tq_deq_b{b}"] = tq.dequantize(c)
    out[f"tq_deq_shrunk_b{b}"] = tq.dequantize(c, shrinkage=2 / np.pi)
    out[f"tq_size_bits_b{b}"] = np.array(tq.compressed_size_bits(100))
    out[f"tq_ratio_b{b}"] = np.array(tq.compression_ratio())

kv = KVCacheCompressor(D, 3, 3, seed=42)
kk = np.random.default_rng(31).standard_normal((1, 2, 16, D))
vv = np.random.default_rng(32).standard_normal((1, 2, 16, D))
cc = kv.compress(kk, vv)
kh, vh = kv.decompress(cc)
out["kv_k"], out["kv_v"], out["kv_k_hat"], out["kv_v_hat"] = kk, vv, kh, vh
out["kv_k_idx_l0h1"] = cc.k_compressed[0][1].mse_indices.astype(np.uint8)
out["kv_k_signs_l0h1"] = cc.k_compressed[0][1].qjl_signs
out["kv_v_idx_l0h1"] = cc.v_indices[0][1].astype(np.uint8)
out["kv_v_norms_l0h1"] = cc.v_norms[0][1]
ms = kv.memory_stats(1024, 32, 8)
out["kv_memory_stats"] = np.array([ms["original_mb"], ms["compressed_mb"], ms["compression_ratio"],
                                   ms["k_bits_per_value"], ms["v_bits_per_value"]], dtype=np.float64)

# ---- host packing ---------------------------------------------------------
sg = np.where(np.random.default_rng(41).random((3, 128)) > 0.5, 1, -1).astype(np.int8)
out["pack_signs_in"] = sg
out["pack_signs_out"] = utils.pack_bits(sg)
out["pack_signs_d5_out"] = utils.pack_bits(sg[0, :5])
for b in (1, 2, 3, 4):
    ii = np.random.default_rng(50 + b).integers(0, 1 << b, size=(3, 40))
    out[f"pack_idx_in_b{b}"] = ii.astype(np.uint8)
    out[f"pack_idx_out_b{b}"] = utils.pack_indices(ii, b)
fp = utils.memory_footprint_bytes(1000, 128, 3)
out["footprint_1000_128_3"] = np.array([fp["mse_indices_bytes"], fp["qjl_signs_bytes"], fp["norms_bytes"],
                                        fp["total_bytes"], fp["original_fp16_bytes"]], dtype=np.int64)

# ---- outlier-channel split (fractional bit rates) ----------------------------
from turboquant.outlier import OutlierTurboQuant, _compute_channel_split  # noqa: E402

out["outlier_split_args"] = np.array([[128, 2.5], [128, 3.5], [128, 3.25], [64, 2.5], [100, 3.5], [128, 3.0]])
out["outlier_split_vals"] = np.array([_compute_channel_split(int(d_), b_) for d_, b_ in out["outlier_split_args"]],
                                     dtype=np.int64)
xo = np.random.default_rng(77).standard_normal((6, D))
xo[2] = 0.0
xo[4] *= 25.0
out["outlier_x"] = xo
for tb in (2.5, 3.5):
    oq = OutlierTurboQuant(D, tb, seed=42)
    tag = f"outlier_{str(tb).replace('.', 'p')}"
    cv = oq.quantize(xo)
    out[f"{tag}_oidx"], out[f"{tag}_onorm"] = cv.outlier_indices.astype(np.uint8), cv.outlier_norms
    out[f"{tag}_nidx"], out[f"{tag}_nnorm"] = cv.normal_indices.astype(np.uint8), cv.normal_norms
    out[f"{tag}_signs"], out[f"{tag}_rnorm"] = cv.qjl_signs, cv.residual_norms
    out[f"{tag}_deq"] = oq.dequantize(cv)
    c1 = oq.quantize(xo[1])
    out[f"{tag}_single_deq"] = oq.dequantize(c1)
    out[f"{tag}_meta"] = np.array([oq.n_outlier, oq.high_bits, oq.n_normal, oq.low_bits, oq.effective_bits,
                                   oq.compression_ratio(), oq.compression_ratio(32)])

# ---- temporal decay: 3-bit block -> 2-bit (benchmarks/temporal_decay_prototype.py:93-125) ----
sys.path.insert(0, os.path.join(ref_root, "benchmarks"))
import temporal_decay_prototype as tdp  # noqa: E402

out["decay_c3"], out["decay_c2"] = tdp.CENTROIDS_3BIT, tdp.CENTROIDS_2BIT
out["decay_mid3"], out["decay_mid2"] = tdp.MIDPOINTS_3BIT, tdp.MIDPOINTS_2BIT
rd = np.random.default_rng(91)
yd = rd.standard_normal((48, D))
yd /= np.linalg.norm(yd, axis=1, keepdims=True)
i3 = np.stack([tdp.quantize_3bit(r) for r in yd])
n3 = np.abs(rd.standard_normal(48)) * 10.0
n3[5] = 0.0
out["decay_idx3"], out["decay_norm3"] = i3, n3
rq = [tdp.requantize_3to2(i3[r], n3[r]) for r in range(48)]
out["decay_idx2"] = np.stack([r_[0] for r_ in rq])
out["decay_norm2"] = np.array([r_[1] for r_ in rq])
out["decay_deq3"] = np.stack([tdp.dequantize_3bit(i3[r], n3[r]) for r in range(48)])
out["decay_deq2"] = np.stack([tdp.dequantize_2bit(out["decay_idx2"][r], out["decay_norm2"][r]) for r in range(48)])

# ---- BASELINE config 1: composition of reference functions ----------------
X = np.random.default_rng(0).standard_normal((4096, D)).astype(np.float32)
sd = np.random.default_rng(1).choice([-1.0, 1.0], size=D)
ones = np.ones(D)
cent = codebook.optimal_centroids(3, D)
nrm = np.linalg.norm(X.astype(np.float64), axis=1)
Y = rotation.apply_fast_rotation_batch(X.astype(np.float64) / nrm[:, None], sd, ones, D)
I = codebook.nearest_centroid_indices(Y, cent)
yh = cent[I]
yh = yh / np.linalg.norm(yh, axis=1, keepdims=True)
xh = np.stack([rotation.apply_fast_rotation_transpose(r, sd, ones, D) for r in yh[:64]]) * nrm[:64, None]
xh_all_rot = yh * nrm[:, None]
out["c1_signs"] = sd
out["c1_idx_first64"] = I[:64].astype(np.uint8)
out["c1_idx_hist"] = np.bincount(I.ravel(), minlength=8)
out["c1_idx_rowsum"] = I.sum(axis=1).astype(np.int64)
out["c1_norms"] = nrm
out["c1_deq_first64"] = xh
# rotation is orthogonal, so the MSE over all rows is the rotated-domain MSE
out["c1_mse"] = np.array(np.mean((xh_all_rot - Y * nrm[:, None]) ** 2))

path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "reference_vectors.npz")
np.savez_compressed(path, **out)
print("wrote", path, os.path.getsize(path), "bytes,", len(out), "arrays")
