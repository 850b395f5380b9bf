"""The benchmark configurations as they are specified, against the oracle.

Configs 3, 4 and 5 at their full sizes (decode attention at batch 16 x 32768 tokens, the asymmetric
q8_0-style K + turbo2 V decode at 4 x 131072 tokens with the +6 bias and Sparse V, the 65536 x 2048
estimator tile) on sampled (batch, kv-head) groups, query rows and key columns, plus config 4's
combination at a reduced size on every group, a hand-built Sparse-V case whose skipped set and output
are known in closed form, and literal q8_0 blocks.

Tolerances are those of test_gpu_attention.py: fp16 operands into the MFMA, fp32 accumulation ->
max abs error <= 2e-3 * max|reference| per query row."""
import numpy as np
import pytest

import tq_oracle as O
import turboquant_plus_amd as tqa
from turboquant_plus_amd import _lib as L

pytestmark = pytest.mark.gpu
D = 128


def np_(t):
    return t.detach().cpu().numpy()


def assert_close(got, ref, rel=2e-3):
    err = np.abs(got - ref).max(axis=-1)
    bound = rel * np.abs(ref).max(axis=-1)
    assert np.all(err <= bound), f"max err/bound = {(err / bound).max():.3f}"


def synth_kv(heads, tokens, seed, outliers):
    """N(0,1) fp16 [heads, tokens, 128] made on the device; `outliers` fixed channels per head x15."""
    tt = L.torch()
    g = tt.Generator(device="cuda").manual_seed(seed)
    x = tt.randn((heads, tokens, D), generator=g, device="cuda", dtype=tt.float32)
    for h in range(heads if outliers else 0):
        ch = np.random.default_rng(1000 + h).choice(D, size=outliers, replace=False)
        x[h][:, tt.as_tensor(ch, device="cuda")] *= 15.0
    return x.to(tt.float16)


def sharpening_bias(B, Hq, N, n_pos, seed):
    """+6 on n_pos random key positions per (batch, query head), fp32 [B, Hq, N]."""
    rng = np.random.default_rng(seed)
    bias = np.zeros((B, Hq, N), dtype=np.float32)
    for b in range(B):
        for h in range(Hq):
            bias[b, h, rng.choice(N, size=n_pos, replace=False)] = 6.0
    return bias


def group_reference(q_group, k_rot, v_rot, vc, scale, n_splits, tau, bias_group):
    o, skip, below = O.decode_attention(q_group, k_rot, v_rot, scale, n_splits=n_splits, sparse_v_tau=tau,
                                        logit_bias=bias_group)
    return O.rotate_fast(o, vc.signs1, vc.signs2, D, transpose=True), skip, below


# ---- config 4: q8_0-style K + turbo2 V + bias + Sparse V ----------------------------------------------

def run_config4(B, Hq, Hkv, N, n_splits, groups, taus=(0.0, 1e-6)):
    tt = L.torch()
    G = Hq // Hkv
    vc = tqa.TurboCodec(2, seed=542)
    perk = int(L.lib().tq_q8_0_bytes(1, N))
    perv = tqa.packed_bytes(2, 1, N)
    kq = tt.empty(B * Hkv * perk, dtype=tt.uint8, device="cuda")
    vp = tt.empty(B * Hkv * perv, dtype=tt.uint8, device="cuda")
    for s in range(B * Hkv):
        kq[s * perk:(s + 1) * perk] = tqa.q8_0_store(synth_kv(1, N, 400 + s, outliers=4))[0]
        vc.store(synth_kv(1, N, 500 + s, outliers=0), kind="v", out=vp[s * perv:(s + 1) * perv])
    q = np.random.default_rng(7).standard_normal((B, Hq, D)).astype(np.float16)
    bias = sharpening_bias(B, Hq, N, 64, seed=8)
    bias_d = tt.from_numpy(bias).cuda()
    scale = 1 / np.sqrt(D)
    outs = {}
    for tau in taus:
        attn = tqa.DecodeAttention(None, vc, B, Hq, Hkv, N, n_splits=n_splits, sparse_v_tau=tau)
        outs[tau] = (np_(attn(q, kq, vp, bias=bias_d)).copy(), attn.skip_rate() if tau else 0.0, attn.params.n_splits)
    skip_sum = {tau: 0.0 for tau in taus}
    for s in groups:
        b, h = divmod(s, Hkv)
        qq, ss = tqa.q8_0_unpack(kq[s * perk:(s + 1) * perk], 1, N)
        k_hat = O.q8_0_dequantize(np_(qq)[0], np_(ss)[0])
        vi, vg = vc.unpack_codes(vp[s * perv:(s + 1) * perv], 1, N, kind="v")
        v_rot = O.turbo_decode_rotated(np_(vi)[0], np_(vg)[0].astype(np.float64), vc.centroids)
        qs = q[b, h * G:(h + 1) * G].astype(np.float64)            # q8_0-style K is not rotated
        for tau in taus:
            out, _, splits = outs[tau]
            ref, skip, _ = group_reference(qs, k_hat, v_rot, vc, scale, splits, tau, bias[b, h * G:(h + 1) * G])
            assert_close(out[b, h * G:(h + 1) * G], ref)
            skip_sum[tau] += skip
    return outs, skip_sum


def test_config4_combination_reduced_every_group():
    B, Hq, Hkv, N = 2, 8, 2, 4096 + 64
    groups = list(range(B * Hkv))
    outs, skip_sum = run_config4(B, Hq, Hkv, N, 16, groups, taus=(0.0, 1e-6, 1e-3))
    for tau in (1e-6, 1e-3):
        rate, ref = outs[tau][1], skip_sum[tau] / len(groups)
        assert abs(rate - ref) <= 0.02 * max(ref, 1e-3) + 1e-4, (tau, rate, ref)
    # tau = 1e-6 drops weights that cannot move the output beyond fp32 noise
    np.testing.assert_allclose(outs[1e-6][0], outs[0.0][0], rtol=0, atol=1e-4 * np.abs(outs[0.0][0]).max())


def test_config4_full_size_as_specified():
    """B 4, 32 query heads on 8 KV heads, context 131072, default split count, +6 bias on 64 positions per
    head, tau 1e-6: outputs of the dense and the Sparse-V step on every group against the oracle, and the
    kernel's skip count against the oracle's count over all 32 groups."""
    B, Hq, Hkv, N = 4, 32, 8, 131072
    groups = list(range(B * Hkv))
    outs, skip_sum = run_config4(B, Hq, Hkv, N, None, groups)
    assert outs[0.0][2] == 128                                       # the benchmark's split count
    rate, ref = outs[1e-6][1], skip_sum[1e-6] / len(groups)
    print(f"\nconfig 4 full size: kernel skip rate {rate:.5f}, oracle {ref:.5f}")
    assert abs(rate - ref) <= 0.02 * max(ref, 1e-3) + 1e-4, (rate, ref)


# ---- config 3: turbo3 K/V decode at full size -------------------------------------------------------------

def test_config3_full_size_sampled_groups():
    """B 16, 32 query heads on 8 KV heads, context 32768, default split count (32: two workgroups of 16
    wavefronts per group, merged by the few-partials kernel): six sampled (batch, kv-head) groups."""
    tt = L.torch()
    B, Hq, Hkv, N, bits = 16, 32, 8, 32768, 3
    kc, vc = tqa.TurboCodec(bits, seed=42), tqa.TurboCodec(bits, seed=542)
    per = tqa.packed_bytes(bits, 1, N)
    kp = tt.empty(B * Hkv * per, dtype=tt.uint8, device="cuda")
    vp = tt.empty_like(kp)
    for b in range(B):
        kc.store_kv(vc, synth_kv(Hkv, N, 100 + b, outliers=4), synth_kv(Hkv, N, 200 + b, outliers=0),
                    out_k=kp[b * Hkv * per:(b + 1) * Hkv * per], out_v=vp[b * Hkv * per:(b + 1) * Hkv * per])
    q = np.random.default_rng(3).standard_normal((B, Hq, D)).astype(np.float16)
    attn = tqa.DecodeAttention(kc, vc, B, Hq, Hkv, N)
    assert attn.params.n_splits == 32
    out = np_(attn(q, kp, vp))
    assert np.isfinite(out).all()
    q_rot = O.rotate_fast(q.astype(np.float64), kc.signs1, kc.signs2, D)
    for s in (0, 7, 8, 63, 100, 127):
        b, h = divmod(s, Hkv)
        ki, kg = kc.unpack_codes(kp[s * per:(s + 1) * per], 1, N, kind="k")
        vi, vg = vc.unpack_codes(vp[s * per:(s + 1) * per], 1, N, kind="v")
        k_rot = O.turbo_decode_rotated(np_(ki)[0], np_(kg)[0].astype(np.float64), kc.centroids)
        v_rot = O.turbo_decode_rotated(np_(vi)[0], np_(vg)[0].astype(np.float64), vc.centroids)
        ref, _, _ = group_reference(q_rot[b, 4 * h:4 * h + 4], k_rot, v_rot, vc, 1 / np.sqrt(D), 1, 0.0, None)
        assert_close(out[b, 4 * h:4 * h + 4], ref)


# ---- config 5: the estimator tile at full size ---------------------------------------------------------------

def test_config5_full_size_sampled_rows_and_columns():
    """65536 keys (3-bit codes + QJL sketch, Gaussian projection seed 2, fp16 residual norm) x 2048 fp16
    queries: eight query rows against all keys and all queries against 96 key columns, the regression slope of
    the sketch's correction term on the true residual inner product (1 only for the scale sqrt(pi/2)/d), and
    the bias of the whole estimate."""
    tt = L.torch()
    nk, nq = 65536, 2048
    g = tt.Generator(device="cuda").manual_seed(11)
    keys = tt.randn((nk, D), generator=g, device="cuda", dtype=tt.float32)
    qs = tt.randn((nq, D), generator=g, device="cuda").to(tt.float16)
    codec = tqa.TurboCodec(3, seed=42, projection="gaussian", projection_seed=2)
    packed, sbits, rn = codec.store_qjl(keys)
    logits = codec.score_tile(qs, packed, sbits, rn, nk)
    assert tuple(logits.shape) == (nq, nk)
    idx, gn = codec.unpack_codes(packed, 1, nk)
    idx, gn = np_(idx)[0], np_(gn)[0].astype(np.float64)
    z = np.unpackbits(np_(sbits), axis=1, bitorder="little")[:, :D].astype(np.float64) * 2 - 1
    rnorm = np_(rn).astype(np.float64)
    qh, kh = np_(qs).astype(np.float64), np_(keys).astype(np.float64)
    rot = lambda a: O.rotate_fast(a, codec.signs1, codec.signs2, D)
    rows = [0, 1, 31, 32, 511, 512, 1000, 2047]
    ref_rows = O.score_tile(qh[rows], idx, gn, codec.centroids, rot, codec.S, z, rnorm, codec.projection_scale)
    bar = 2e-3 * np.linalg.norm(qh, axis=1).max() * np.linalg.norm(kh, axis=1).max() / np.sqrt(D) * 4
    assert np.abs(np_(logits[rows]) - ref_rows).max() <= bar
    cols = np.random.default_rng(5).choice(nk, size=96, replace=False)
    cols.sort()
    ref_cols = O.score_tile(qh, idx[cols], gn[cols], codec.centroids, rot, codec.S, z[cols], rnorm[cols],
                            codec.projection_scale)
    got_cols = np_(logits[:, tt.as_tensor(cols, device="cuda")])
    assert np.abs(got_cols - ref_cols).max() <= bar
    # correction term = logits - <R q, g c[idx]> regressed on <q, residual>
    k_mse = O.turbo_decode(idx[cols], gn[cols], codec.centroids, codec.signs1, codec.signs2)
    resid = kh[cols] - k_mse
    corr = got_cols - qh @ k_mse.T
    true = qh @ resid.T
    slope = (corr * true).sum() / (true * true).sum()
    assert abs(slope - 1.0) < 0.05, slope
    err = got_cols - qh @ kh[cols].T
    assert abs(err.mean()) < 4 * err.std() / np.sqrt(err.size) + 1e-3


# ---- Sparse V: the hand-built case --------------------------------------------------------------------------------

def test_sparse_v_hand_built_case_on_the_gpu():
    """Zero queries, logits given by the bias as multiples of ln 10 (weights are powers of ten), N = 256 in two
    splits of two tiles, tau = 1e-2.  Head 0: kept set {0, 1, 64, 65, 128, 129, 192} (a position kept against the
    running maximum that the split's final maximum would drop; a later position with a larger logit skipped; a
    split that starts from its own maximum).  Head 1: all logits equal, nothing skipped, output = mean of V.
    Heads 2, 3 repeat head 0 so that the count is 3 * 249 of 4 * 256."""
    tt = L.torch()
    N, ln10 = 256, np.log(10.0)
    e = np.full(N, -30.0)
    for pos, val in {0: 0, 1: -1, 2: -3, 64: 3, 65: 2, 66: 0.5, 128: 1, 129: -0.5, 192: 1, 193: -1.5}.items():
        e[pos] = val
    kept = [0, 1, 64, 65, 128, 129, 192]
    bias = np.stack([e * ln10, np.zeros(N), e * ln10, e * ln10]).astype(np.float32)[None]        # [1, 4, N]
    rng = np.random.default_rng(0)
    k = rng.standard_normal((1, N, D)).astype(np.float16)
    v = rng.standard_normal((1, N, D)).astype(np.float32)
    v[0, 0] *= 300.0        # weight 1 next to weight 1000 at pos 64: large rows make the kept set visible in the output
    v[0, 128] *= 30.0       # weight 10
    v = v.astype(np.float16)
    kc, vc = tqa.TurboCodec(3, seed=42), tqa.TurboCodec(3, seed=542)
    kp, vp = kc.store(k, kind="k"), vc.store(v, kind="v")
    v_hat = np_(vc.load(vp, 1, N, kind="v", domain="original"))[0].astype(np.float64)
    q = np.zeros((1, 4, D), dtype=np.float16)
    attn = tqa.DecodeAttention(kc, vc, 1, 4, 1, N, n_splits=2, sparse_v_tau=1e-2)
    out = np_(attn(q, kp, vp, bias=tt.from_numpy(bias).cuda()))[0]
    w = 10.0 ** e
    expect0 = (w[kept, None] * v_hat[kept]).sum(0) / w.sum()
    for h in (0, 2, 3):
        assert_close(out[h][None], expect0[None])
    assert_close(out[1][None], v_hat.mean(0)[None], rel=3e-3)
    cnt = attn.skip.cpu().numpy()
    assert cnt.tolist() == [3 * (N - len(kept)), 4 * N]
    # the same logits with the final-maximum rule or one maximum carried over both splits give other outputs
    for wrong in ([64, 65, 128, 129, 192], [0, 1, 64, 65]):
        other = (w[wrong, None] * v_hat[wrong]).sum(0) / w.sum()
        assert np.abs(other - expect0).max() > 0.05 * np.abs(expect0).max()


# ---- q8_0-style blocks: literals ----------------------------------------------------------------------------------------

@pytest.mark.parametrize("kind", ["k", "v"])
def test_q8_0_literal_blocks_on_the_gpu(kind):
    """The hand-made blocks of tests/test_oracle_math.py::test_q8_0_literal_blocks through both store paths:
    ties away from zero, the largest float below one half, a zero block, the division by the unrounded scale."""
    x = np.zeros((1, 70, D), dtype=np.float32)
    b0 = [-127.0, 0.5, -0.5, 1.5, -1.5, 2.5, -2.5, 126.5, -126.5, 0.49999997, -0.49999997, 0.50000006, 3.0, -0.0, 100.25, -100.75]
    q0 = [-127, 1, -1, 2, -2, 3, -3, 127, -127, 0, 0, 1, 3, 0, 100, -101]
    d2 = np.float32(1.0) + np.float32(2.0 ** -12)
    for t in (0, 69):                                  # first row, and a row of the ragged second 64-token tile
        x[0, t, :16] = b0
        x[0, t, 64:68] = [np.float32(127.0) * d2, 100.5, 0.5, -100.5]
        x[0, t, 96:100] = [-63.5, 0.25, 0.75, -0.25]
    packed, _, _ = tqa.q8_0_store(x, kind=kind)
    q, s = tqa.q8_0_unpack(packed, 1, 70, kind=kind)
    q, s = np_(q)[0], np_(s)[0]
    for t in (0, 69):
        assert q[t, :16].tolist() == q0 and not q[t, 16:64].any()
        assert q[t, 64:68].tolist() == [127, 100, 0, -100]
        assert q[t, 96:100].tolist() == [-127, 1, 2, -1]
        assert s[t].tolist() == [1.0, 0.0, 1.0, 0.5]
    assert not q[1:69].any() and not s[1:69].any()
    # fp16 input (the fast store kernels): every literal that fp16 holds exactly
    xh = np.zeros((1, 128, D), dtype=np.float16)
    xh[0, 5, :9] = b0[:9]
    xh[0, 5, 32:36] = [254.0, 1.0, 3.0, -5.0]          # d = 2: 0.5 -> 1, 1.5 -> 2, -2.5 -> -3
    xh[0, 127, 96:100] = [-63.5, 0.25, 0.75, -0.25]
    packed, _, _ = tqa.q8_0_store(xh, kind=kind)
    q, s = tqa.q8_0_unpack(packed, 1, 128, kind=kind)
    q, s = np_(q)[0], np_(s)[0]
    assert q[5, :9].tolist() == q0[:9] and q[5, 32:36].tolist() == [127, 1, 2, -3]
    assert q[127, 96:100].tolist() == [-127, 1, 2, -1] and s[5].tolist() == [1.0, 2.0, 0.0, 0.0]
    qo, so = O.q8_0_quantize(xh[0])
    assert np.array_equal(q, qo) and np.array_equal(s.astype(np.float16), so)
