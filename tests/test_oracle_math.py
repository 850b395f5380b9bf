"""What the mathematics fixes about the oracle, independent of any fixture:
library routines, closed forms, brute force on small inputs, invariants.
Mirrors the known-answer checks of the reference's tests/test_rotation.py,
test_codebook.py, test_qjl.py and test_utils.py."""
import numpy as np
import pytest
import scipy.linalg

import tq_oracle as O


@pytest.mark.parametrize("n", [1, 2, 8, 64, 128])
def test_fwht_is_scipy_hadamard(n):
    x = np.random.default_rng(n).standard_normal((5, n))
    ref = x @ (scipy.linalg.hadamard(n) / np.sqrt(n)).T
    np.testing.assert_allclose(O.fwht(x), ref, atol=1e-12)
    np.testing.assert_allclose(O.fwht(O.fwht(x)), x, atol=1e-12)


def test_fwht_rejects_non_pow2():
    with pytest.raises(ValueError, match="power of 2"):
        O.fwht(np.zeros(12))


def test_sylvester_matches_scipy():
    for n in (1, 2, 4, 16, 128):
        assert np.array_equal(O.sylvester_hadamard(n), scipy.linalg.hadamard(n))
    with pytest.raises(ValueError):
        O.sylvester_hadamard(6)


def test_fast_rotation_is_explicit_matrix():
    rng = np.random.default_rng(5)
    s1, s2, pd = O.sign_diagonals(128, rng)
    R = np.diag(s2) @ (scipy.linalg.hadamard(128) / np.sqrt(128)) @ np.diag(s1)
    x = rng.standard_normal((7, 128))
    np.testing.assert_allclose(O.rotate_fast(x, s1, s2, pd), x @ R.T, atol=1e-12)
    np.testing.assert_allclose(O.rotate_fast(x, s1, s2, pd, transpose=True), x @ R, atol=1e-12)
    # padded, truncated case: d = 100 inside 128
    x = rng.standard_normal((3, 100))
    full = np.zeros((3, 128)); full[:, :100] = x
    np.testing.assert_allclose(O.rotate_fast(x, s1, s2, pd), (full @ R.T)[:, :100], atol=1e-12)


@pytest.mark.parametrize("d", [1, 8, 64, 128])
def test_haar_is_rotation(d):
    q = O.haar_rotation(d, np.random.default_rng(d))
    np.testing.assert_allclose(q @ q.T, np.eye(d), atol=1e-10)
    assert np.linalg.slogdet(q)[0] > 0
    with pytest.raises(ValueError):
        O.haar_rotation(0, np.random.default_rng(0))


def test_centroid_closed_forms():
    for d in (64, 128, 256):
        np.testing.assert_allclose(O.centroids_for(1, d), [-np.sqrt(2 / (np.pi * d)), np.sqrt(2 / (np.pi * d))], atol=1e-15)
        np.testing.assert_allclose(O.centroids_for(2, d), np.array([-1.51, -0.453, 0.453, 1.51]) / np.sqrt(d), atol=1e-15)
    # textbook Max (1960) 8-level unit-Gaussian quantiser
    max8 = np.array([0.2451, 0.7560, 1.3439, 2.1520])
    c = O.centroids_for(3, 128) * np.sqrt(128)
    np.testing.assert_allclose(c[4:], max8, atol=2e-4)
    np.testing.assert_allclose(c, -c[::-1], atol=1e-12)


def test_cond_mean_closed_forms():
    assert abs(O.gauss_cond_mean(1.0, 0.0, np.inf) - np.sqrt(2 / np.pi)) < 1e-12
    assert abs(O.gauss_cond_mean(1.0, -1.0, 1.0)) < 1e-12
    assert O.gauss_cond_mean(1.0, 40.0, np.inf) == 41.0
    assert O.gauss_cond_mean(1.0, -np.inf, -40.0) == -41.0
    assert O.gauss_cond_mean(1.0, 40.0, 41.0) == 40.5
    # numeric integration of x*pdf over [a,b] / mass
    xs = np.linspace(-0.3, 0.7, 200001)
    pdf = np.exp(-xs ** 2 / (2 * 0.25)) / np.sqrt(2 * np.pi * 0.25)
    num = np.trapezoid(xs * pdf, xs) / np.trapezoid(pdf, xs)
    assert abs(O.gauss_cond_mean(0.5, -0.3, 0.7) - num) < 1e-9


@pytest.mark.parametrize("b", [1, 2, 3, 4])
def test_nearest_index_is_argmin(b):
    c = O.centroids_for(b, 128)
    v = np.random.default_rng(b).standard_normal(500) / np.sqrt(128)
    brute = np.argmin(np.abs(v[:, None] - c[None, :]), axis=1)
    assert np.array_equal(O.nearest_index(v, c), brute)
    # tie rule: exactly on a midpoint -> lower index; far outside -> clamped
    mid = O.midpoints(c)
    assert np.array_equal(O.nearest_index(mid, c), np.arange(len(mid)))
    assert O.nearest_index(np.array([-9.0, 9.0]), c).tolist() == [0, len(c) - 1]


def test_qjl_orthogonal_and_unbiased():
    for d in (64, 128):
        q = O.QJLRef(d, seed=123)
        assert np.linalg.norm(q.S @ q.S.T - np.eye(d), "fro") < 1e-12
    q = O.QJLRef(128, seed=5)
    rng = np.random.default_rng(0)
    x, y = rng.standard_normal(128), rng.standard_normal(128)
    # E||x_hat||^2 = (pi/2)||x||^2 holds exactly for orthogonal S and +-1 signs
    z, n = q.quantize(x)
    assert abs(np.linalg.norm(q.dequantize(z, n)) ** 2 - (np.pi / 2) * n ** 2) < 1e-9
    # unbiasedness over many projection seeds
    est = []
    for s in range(300):
        qq = O.QJLRef(128, seed=s)
        z, n = qq.quantize(x)
        est.append(qq.dequantize(z, n) @ y)
    se = np.std(est) / np.sqrt(len(est))
    assert abs(np.mean(est) - x @ y) < 4 * se
    z, n = q.quantize(np.zeros(128))
    assert n == 0 and set(np.unique(z)) == {1}


def test_pack_literals():
    # reference tests/test_utils.py literals: 8 signs -> one byte, MSB first
    assert O.pack_sign_bits(np.array([1, -1, 1, 1, -1, -1, 1, -1], dtype=np.int8)).tolist() == [0b10110010]
    assert O.pack_sign_bits(np.ones(128, dtype=np.int8)).shape == (16,)
    assert O.pack_index_stream(np.array([3, 0, 1, 2]), 2).tolist() == [0b11000110]
    assert O.pack_index_stream(np.array([5, 2]), 3).tolist() == [0b10101000]
    with pytest.raises(ValueError, match="bit_width must be 1-8"):
        O.pack_index_stream(np.array([0]), 9)
    assert O.TurboRef(128, 3).compressed_size_bits(100) == 100 * (128 * 3 + 32)


def test_polar_invariants():
    pq = O.PolarRef(128, 3, seed=1)
    x = np.random.default_rng(2).standard_normal((16, 128))
    idx, n = pq.quantize(x)
    assert idx.min() >= 0 and idx.max() < 8
    np.testing.assert_allclose(pq.dequantize(*pq.quantize(3.0 * x)), 3.0 * pq.dequantize(idx, n), rtol=1e-12)
    assert np.all(pq.dequantize(*pq.quantize(np.zeros((2, 128)))) == 0)
    xu = x / np.linalg.norm(x, axis=1, keepdims=True)
    mse = np.mean(np.sum((pq.dequantize(*pq.quantize(xu)) - xu) ** 2, axis=1))
    assert mse < 2 * 0.03
    # wht mode: same contract, different rotation
    pw = O.PolarRef(128, 3, seed=1, rotation="wht")
    mse = np.mean(np.sum((pw.dequantize(*pw.quantize(xu)) - xu) ** 2, axis=1))
    assert mse < 2 * 0.03


@pytest.mark.parametrize("bits", [2, 3, 4])
@pytest.mark.parametrize("kind", ["k", "v"])
def test_device_layout_roundtrip_and_placement(bits, kind):
    rng = np.random.default_rng(bits)
    T = 256
    idx = rng.integers(0, 1 << bits, size=(T, 128)).astype(np.uint8)
    g = rng.standard_normal(T).astype(np.float16)
    buf = O.layout_pack(idx, g, bits, kind)
    assert buf.dtype == np.uint8 and buf.size == 2 * O.block_bytes(bits) == T * (16 * bits + 2)
    i2, g2 = O.layout_unpack(buf, bits, kind)
    assert np.array_equal(i2, idx) and np.array_equal(g2.view(np.uint16), g.view(np.uint16))
    # one-hot placement: a single non-zero code lands where the layout says
    for tok, dim in [(77, 45), (5, 31), (64, 127), (127, 94), (0, 0)]:
        one = np.zeros((128, 128), dtype=np.uint8)
        one[tok, dim] = (1 << bits) - 1
        b = O.layout_pack(one, np.zeros(128, dtype=np.float16), bits, kind)
        words = b[:128 * 16 * bits].view("<u4").reshape(bits, 128, 4)
        if kind == "k":
            row, pair, half = tok, dim // 2, dim % 2
        else:
            tp = (tok & 63) // 2
            row, pair, half = (tok & 64) | (dim & 63), 4 * (tp // 2) + 2 * (dim >> 6) + tp % 2, tok % 2
        value = ((1 << bits) - 1) << (bits * half)
        rowwords = words[:, row, :].reshape(-1)
        expect = np.zeros(4 * bits, dtype=np.uint64)
        grp, k = pair // 16, pair % 16
        if bits == 4:
            expect[4 * (k // 4) + grp] = value << (8 * (k % 4))
        elif bits == 2:
            expect[4 * (k // 8) + grp] = value << (4 * (k % 8))
        elif k < 12:
            expect[4 * (k // 4) + grp] = value << (6 * (k % 4))
        else:
            tail = value << (6 * (k - 12))
            for part in range(3):
                expect[4 * part + grp] = ((tail >> (8 * part)) & 0xFF) << 24
        assert np.array_equal(rowwords.astype(np.uint64), expect)
        assert np.count_nonzero(words) == np.count_nonzero(expect)


def test_turbo_encode_consistency():
    rng = np.random.default_rng(3)
    s1, s2, _ = O.sign_diagonals(128, rng)
    cent = O.centroids_for(4, 128)
    x = rng.standard_normal((64, 128))
    x[3] = 0
    idx, g, y = O.turbo_encode(x, s1, s2, cent)
    assert g.dtype == np.float16 and g[3] == 0
    # corrected norm: reconstruction has the original norm up to fp16 rounding
    rec = O.turbo_decode(idx, g, cent, s1, s2)
    np.testing.assert_allclose(np.linalg.norm(rec, axis=1), np.linalg.norm(x, axis=1), rtol=1e-3)
    assert np.all(rec[3] == 0)
    # same indices as the class in wht mode built from the same signs
    n_bad, n_inadm = O.boundary_band_mismatches(y, idx, cent)
    assert (n_bad, n_inadm) == (0, 0)
    bad = idx.copy(); bad[0, 0] ^= 1
    assert O.boundary_band_mismatches(y, bad, cent)[1] == 1


def test_q8_0_textbook():
    x = np.random.default_rng(4).standard_normal((5, 128)).astype(np.float32)
    x[0, :32] = 0
    q, s = O.q8_0_quantize(x)
    assert q.dtype == np.int8 and s.shape == (5, 4) and s.dtype == np.float16
    assert np.all(q[0, :32] == 0) and s[0, 0] == 0
    assert np.abs(q).max() == 127
    err = np.abs(O.q8_0_dequantize(q, s) - x)
    assert err.max() <= np.abs(x).reshape(5, 4, 32).max(-1).max() / 127 * 0.51 + 1e-3


def test_q8_0_literal_blocks():
    """ggml's quantize_row_q8_0 written out on four hand-made 32-value blocks: d = amax/127 kept in fp32 for
    the division (id = 1/d, x*id), stored as fp16; q = roundf(x*id), i.e. halves go away from zero."""
    x = np.zeros((1, 128), dtype=np.float32)
    # block 0: amax 127 -> d = 1, q = roundf(x).  Ties at +-0.5, +-1.5, +-2.5 (banker's rounding would give
    # 0, 2, 2), values just either side of a half, the extreme on the negative side.
    b0 = [-127.0, 0.5, -0.5, 1.5, -1.5, 2.5, -2.5, 126.5, -126.5, 0.49999997, -0.49999997, 0.50000006, 3.0, -0.0, 100.25, -100.75]
    x[0, :len(b0)] = b0
    q0 = [-127, 1, -1, 2, -2, 3, -3, 127, -127, 0, 0, 1, 3, 0, 100, -101]
    # block 1: all zero -> d = 0, id = 0, q = 0
    # block 2: amax = 127 * (1 + 2^-12): d = 1 + 2^-12 in fp32, which fp16 rounds to 1.0.  100.5 / d = 100.4755
    # -> 100 (dividing by the fp16-rounded scale would give 100.5 -> 101); 0.5 / d < 0.5 -> 0 (1 with the
    # rounded scale).
    d2 = np.float32(1.0) + np.float32(2.0 ** -12)
    x[0, 64:68] = [np.float32(127.0) * d2, 100.5, 0.5, -100.5]
    q2 = [127, 100, 0, -100]
    # block 3: amax 63.5 -> d = 0.5: -63.5 -> -127, 0.25 -> 0.5 -> 1, 0.75 -> 1.5 -> 2, -0.25 -> -1
    x[0, 96:100] = [-63.5, 0.25, 0.75, -0.25]
    q3 = [-127, 1, 2, -1]
    q, s = O.q8_0_quantize(x)
    assert q[0, :16].tolist() == q0 and not q[0, 16:64].any()
    assert q[0, 64:68].tolist() == q2 and not q[0, 68:96].any()
    assert q[0, 96:100].tolist() == q3 and not q[0, 100:].any()
    assert s.dtype == np.float16 and s[0].tolist() == [1.0, 0.0, 1.0, 0.5]
    # dequantised value = q * stored (fp16) scale
    np.testing.assert_array_equal(O.q8_0_dequantize(q, s)[0, 96:100], [-63.5, 0.5, 1.0, -0.5])
    np.testing.assert_array_equal(O.q8_0_dequantize(q, s)[0, 64:66], [127.0, 100.0])


def test_decode_attention_closed_forms():
    rng = np.random.default_rng(6)
    q = rng.standard_normal((4, 128))
    v = rng.standard_normal((256, 128))
    # identical keys -> uniform weights -> mean of V
    k = np.tile(rng.standard_normal((1, 128)), (256, 1))
    out, _, _ = O.decode_attention(q, k, v, 0.1)
    np.testing.assert_allclose(out, np.tile(v.mean(0), (4, 1)), atol=1e-12)
    # one dominant key -> its V row
    k = rng.standard_normal((256, 128)) * 1e-3
    k[17] = 50 * q[0]
    out, _, _ = O.decode_attention(q[:1], k, v, 1.0)
    np.testing.assert_allclose(out[0], v[17], atol=1e-9)
    # brute force softmax, and tau = 0 == dense, tau > 0 with splits close to dense
    k = rng.standard_normal((256, 128))
    s = 0.2 * q @ k.T
    p = np.exp(s - s.max(1, keepdims=True)); p /= p.sum(1, keepdims=True)
    dense, _, _ = O.decode_attention(q, k, v, 0.2)
    np.testing.assert_allclose(dense, p @ v, atol=1e-12)
    sp, skip, frac = O.decode_attention(q, k, v, 0.2, n_splits=4, sparse_v_tau=1e-6)
    assert 0 <= skip <= 1 and np.abs(sp - dense).max() < 1e-3
    sp0, skip0, _ = O.decode_attention(q, k, v, 0.2, n_splits=4, sparse_v_tau=0.0)
    assert skip0 == 0 and np.array_equal(sp0, dense)


def _sparse_v_case():
    """Logits are written directly (zero queries, logits = bias) as multiples of ln 10, so every weight
    is a power of ten and the Sparse-V bookkeeping can be done by hand.  N = 256 in 2 splits of two
    64-position tiles each; tau = 1e-2.  Row 0 of the bias:

      split 0, tile 0: pos 0 -> 0 (tile max, weight 1: kept), pos 1 -> -1 (0.1: kept), pos 2 -> -3 (1e-3: skipped)
      split 0, tile 1: pos 64 -> +3 (new running max), pos 65 -> +2 (0.1: kept), pos 66 -> +0.5 (10^-2.5: skipped,
                       although its logit is above that of pos 0, which was kept against the earlier maximum;
                       against the split's final maximum pos 0 and pos 1 would be 1e-3 and 1e-4: skipped)
      split 1, tile 2: pos 128 -> +1 (max of ITS split: kept), pos 129 -> -0.5 (10^-1.5 against the split's own
                       maximum: kept; against a maximum carried over from split 0 it would be 10^-3.5)
      split 1, tile 3: pos 192 -> +1 (equal to the running max: weight 1, kept), pos 193 -> -1.5 (10^-2.5: skipped)
      every other position -> -30 (skipped)

    Row 1 is all zeros: every weight is 1, nothing is skipped, the output is the mean of V."""
    N, ln10 = 256, np.log(10.0)
    e = np.full(N, -30.0)
    for pos, val in {0: 0, 1: -1, 2: -3, 64: 3, 65: 2, 66: 0.5, 128: 1, 129: -0.5, 192: 1, 193: -1.5}.items():
        e[pos] = val
    bias = np.stack([e * ln10, np.zeros(N)])
    kept = [0, 1, 64, 65, 128, 129, 192]
    return N, e, bias, kept


def test_sparse_v_hand_built_case():
    N, e, bias, kept = _sparse_v_case()
    rng = np.random.default_rng(0)
    k = rng.standard_normal((N, 128))
    v = np.zeros((N, 128))
    v[:, 0] = 1.0                       # output[0] = kept weight / total weight
    v[:, 1] = np.arange(N)              # output[1] = weighted mean position of the kept set
    v[:, 2] = rng.standard_normal(N)
    out, skip, below = O.decode_attention(np.zeros((2, 128)), k, v, 0.3, n_splits=2, sparse_v_tau=1e-2,
                                          logit_bias=bias)
    w = 10.0 ** e
    Z = w.sum()
    assert abs(Z - 1124.6111282027869) < 1e-9             # 1000+100+10+10+sqrt(10)+1+1/sqrt(10)+.1+10^-1.5+.001
    assert abs(out[0, 0] - 1121.416227766017 / 1124.6111282027869) < 1e-12
    pos_sum = 1 * 0.1 + 64 * 1000 + 65 * 100 + 128 * 10 + 129 * 10 ** -0.5 + 192 * 10
    assert abs(out[0, 1] - pos_sum / Z) < 1e-9
    assert abs(out[0, 2] - (w[kept] * v[kept, 2]).sum() / Z) < 1e-12
    np.testing.assert_allclose(out[1], v.mean(0), atol=1e-12)
    assert skip == (N - len(kept)) / (2 * N)               # 249 skipped pairs of 512
    # final softmax weights >= tau: 1000/Z and 100/Z only; row 1 has 1/256 < 1e-2 everywhere
    assert below == (254 + 256) / 512
    # the three plausible mistakes give other numbers
    final_max_kept = [64, 65]                              # weights against the split's final maximum
    assert abs(out[0, 0] - w[final_max_kept + [128, 129, 192]].sum() / Z) > 1e-4
    carried_max_kept = [0, 1, 64, 65]                      # one running maximum over both splits
    assert abs(out[0, 0] - w[carried_max_kept].sum() / Z) > 1e-3


def test_sparse_v_threshold_is_strict():
    """weight < tau skips, weight == tau keeps (docs/papers/sparse-v-dequant.md:69-75 `if (attn_weight < 1e-6f)
    continue`): with tau = 1 exactly the positions that hold the running maximum (weight exp(0) = 1) survive."""
    N = 128
    bias = np.zeros((1, N))
    bias[0, [5, 70]] = [2.0, 2.0]       # tile 0: pos 5 is the max; tile 1: pos 70 ties the running max
    bias[0, 100] = 1.0
    v = np.zeros((N, 128)); v[:, 0] = np.arange(N)
    out, skip, _ = O.decode_attention(np.zeros((1, 128)), np.zeros((N, 128)), v, 1.0, n_splits=1, sparse_v_tau=1.0,
                                      logit_bias=bias)
    Z = 2 * np.exp(2.0) + np.exp(1.0) + (N - 3)
    assert abs(out[0, 0] - (5 + 70) * np.exp(2.0) / Z) < 1e-12
    assert skip == (N - 2) / N


def test_sparse_v_split_bounds():
    """Splits are runs of ceil(n_tiles / n_splits) tiles: N = 320 (5 tiles) in 2 splits -> tiles {0,1,2} and {3,4}.
    pos 130 (tile 2) -> +5, pos 190 (tile 2) -> 0, pos 200 (tile 3) -> 0, everything else -30.  Tiles 0 and 1 see
    only -30: every weight there is 1 against the running maximum and is kept (128 positions of negligible
    weight).  Tile 2: 130 kept, 190 (1e-5) and the rest skipped.  Tile 3 opens split 1 with a fresh maximum:
    200 kept (with tiles {0,1} / {2,3,4}, or a carried maximum, it would be 1e-5 and skipped).  Tile 4: all skipped."""
    N, ln10 = 320, np.log(10.0)
    e = np.full(N, -30.0)
    e[130], e[190], e[200] = 5, 0, 0
    v = np.zeros((N, 128)); v[:, 0] = 1.0
    out, skip, _ = O.decode_attention(np.zeros((1, 128)), np.zeros((N, 128)), v, 1.0, n_splits=2, sparse_v_tau=1e-3,
                                      logit_bias=(e * ln10)[None])
    assert skip == (N - 130) / N
    assert abs(out[0, 0] - (1e5 + 1) / (1e5 + 2)) < 1e-12


def test_gaussian_projection_scale_by_slope():
    """QJL with a raw Gaussian matrix: E[S^T sign(S r)] = d sqrt(2/pi) r/|r|, so the reconstruction
    scale * |r| * S^T sign(S r) has regression slope 1 on r only for scale = sqrt(pi/2)/d.  The slope
    sum(<q,r_hat><q,r>) / sum(<q,r>^2) over many keys and queries is 1 within sampling error; the orthogonal
    mode's constant sqrt(pi/2)/sqrt(d) would give sqrt(d) = 11.3."""
    d = 128
    rng = np.random.default_rng(11)
    r = rng.standard_normal((4000, d))
    qv = rng.standard_normal((64, d))
    for mode in ("gaussian", "orthogonal"):
        ql = O.QJLRef(d, seed=2, projection=mode)
        z, n = ql.quantize(r)
        r_hat = ql.dequantize(z, n)
        a, b = qv @ r_hat.T, qv @ r.T
        slope = (a * b).sum() / (b * b).sum()
        assert abs(slope - 1.0) < 0.03, (mode, slope)
    # and the score tile's correction term carries that same constant
    ql = O.QJLRef(d, seed=2, projection="gaussian")
    assert ql.scale == np.sqrt(np.pi / 2) / d
    z, n = ql.quantize(r[:50])
    tile = O.score_tile(qv, np.zeros((50, d), dtype=np.int64), np.zeros(50), np.zeros(8), lambda a: a, ql.S, z, n, ql.scale)
    np.testing.assert_allclose(tile, qv @ ql.dequantize(z, n).T, atol=1e-10)


def test_score_tile_is_dequantised_inner_product():
    rng = np.random.default_rng(8)
    tq = O.TurboRef(128, 4, seed=42, rotation="wht")
    keys = rng.standard_normal((32, 128))
    qs = rng.standard_normal((5, 128))
    c = tq.quantize(keys)
    direct = qs @ tq.dequantize(c).T
    pq = tq.polar_quant
    cent = pq.centroids
    cn = np.linalg.norm(cent[c.mse_indices], axis=1)
    g = c.vector_norms / cn
    tile = O.score_tile(qs, c.mse_indices, g, cent, lambda a: O.rotate_fast(a, pq.s1, pq.s2, pq.pd),
                        tq.qjl.S, c.qjl_signs, c.residual_norms, tq.qjl.scale)
    np.testing.assert_allclose(tile, direct, atol=1e-11)


@pytest.mark.parametrize("bits", [2, 3, 4])
def test_fork_block_layout_formulas(bits):
    """Per-128 block layout of the llama.cpp fork: the extraction formulas printed in
    docs/papers/turbo4-resurrection.md:130-134,169, applied element by element to what fork_blocks_pack wrote, and
    the block sizes the reference prints: 50 B for turbo3 (3.125 bits per value, docs/papers/block-size-experiment.md:33-39),
    68 B for turbo4 (docs/papers/turbo4-resurrection.md:208 "qs[64], maintaining the 68-byte block size"; 4.25 bits
    per value, README.md:43,94), 34 B for turbo2 (2.125)."""
    rng = np.random.default_rng(bits)
    idx = rng.integers(0, 1 << bits, size=(5, 128)).astype(np.uint8)
    g = rng.standard_normal(5).astype(np.float16)
    buf = O.fork_blocks_pack(idx, g, bits)
    assert buf.shape == (5, {2: 34, 3: 50, 4: 68}[bits])
    assert O.fork_block_bytes(bits) * 8 / 128 == {2: 2.125, 3: 3.125, 4: 4.25}[bits]   # the figures the reference prints
    for t in range(5):
        row = buf[t]
        assert row[:2].view(np.float16)[0] == g[t]
        if bits == 4:
            assert row[2] == 0 and row[3] == 0          # the struct's unused rnorm field
        qs = row[4:68] if bits == 4 else row[2:34]
        signs = row[34:50] if bits == 3 else None
        for j in range(128):
            if bits == 4:
                got = (qs[j // 2] >> ((j % 2) * 4)) & 0xF
            else:
                got = (qs[j // 4] >> ((j % 4) * 2)) & 0x3
                if bits == 3 and signs[j // 8] & (1 << (j % 8)):
                    got |= 4
            assert got == idx[t, j]
    i2, g2 = O.fork_blocks_unpack(buf, bits)
    assert np.array_equal(i2, idx) and np.array_equal(g2.view(np.uint16), g.view(np.uint16))
    if bits == 4:                                        # whatever a writer left in rnorm does not reach the codes
        buf[:, 2:4] = 0xA5
        i3, g3 = O.fork_blocks_unpack(buf, bits)
        assert np.array_equal(i3, idx) and np.array_equal(g3.view(np.uint16), g.view(np.uint16))


@pytest.mark.parametrize("bits", [2, 3])
@pytest.mark.parametrize("block_values", [32, 64, 128])
def test_fork_storage_block_sizes(bits, block_values):
    """The fork's earlier storage blocks of 32 (and 64) values, docs/papers/block-size-experiment.md:33-39: "norm(2B) +
    qs(8B) + signs(4B) = 14B per 32" (3.50 bits per value, 4.57x), 26 B per 64 (3.25, 4.92x), 50 B per 128 (3.125,
    5.12x); four blocks of a 128-value group "receive the same corrected norm value" (:13).  The extraction formulas
    are applied by hand inside every block of what fork_blocks_pack wrote."""
    bb = O.fork_block_bytes(bits, block_values)
    if bits == 3:
        assert bb == {32: 14, 64: 26, 128: 50}[block_values]
        assert bb * 8 / block_values == {32: 3.5, 64: 3.25, 128: 3.125}[block_values]
        assert round(16 / (bb * 8 / block_values), 2) == {32: 4.57, 64: 4.92, 128: 5.12}[block_values]
    else:
        assert bb == {32: 10, 64: 18, 128: 34}[block_values]
    n_blocks = 128 // block_values
    assert O.fork_row_bytes(bits, block_values) == n_blocks * bb
    rng = np.random.default_rng(10 * bits + block_values)
    idx = rng.integers(0, 1 << bits, size=(4, 128)).astype(np.uint8)
    g = np.abs(rng.standard_normal(4)).astype(np.float16)
    buf = O.fork_blocks_pack(idx, g, bits, block_values)
    assert buf.shape == (4, n_blocks * bb)
    for t in range(4):
        for b in range(n_blocks):
            blk = buf[t, b * bb:(b + 1) * bb]
            assert blk[:2].view(np.float16)[0] == g[t]                     # the group's norm in every block
            qs = blk[2:2 + block_values // 4]
            signs = blk[2 + block_values // 4:]
            assert len(signs) == (block_values // 8 if bits == 3 else 0)
            for j in range(block_values):
                got = (qs[j // 4] >> ((j % 4) * 2)) & 3
                if bits == 3 and signs[j // 8] & (1 << (j % 8)):
                    got |= 4
                assert got == idx[t, b * block_values + j]
    i2, g2 = O.fork_blocks_unpack(buf, bits, block_values)
    assert np.array_equal(i2, idx) and np.array_equal(g2.view(np.uint16), g.view(np.uint16))
    if block_values == 128:                                                # the default is the per-128 layout
        assert np.array_equal(buf, O.fork_blocks_pack(idx, g, bits))
    with pytest.raises(ValueError):
        O.fork_block_bytes(4, 32)                                          # turbo4 blocks hold 128 values
