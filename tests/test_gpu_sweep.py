"""Seeded random sweeps of the HIP path against the oracle: shapes, dtypes, formats and row kinds that the
hand-picked cases of the other GPU tests do not enumerate.  Every case prints its parameters before it runs, so a
failure names them; the bars are those of the tests the helpers come from (bit-exact codes outside the 1e-6 boundary
band, byte-equal layouts, 2e-3 of the row maximum for attention)."""
import numpy as np
import pytest

import tq_oracle as O
import turboquant_plus_amd as tqa
from turboquant_plus_amd import _lib as L
import test_gpu_attention as TA
import test_gpu_append as TP
from test_gpu_turbo import check_codes, np_

pytestmark = pytest.mark.gpu
D = 128


def _rows(rng, shape, dtype, flavour):
    """Row kinds: Gaussian, K-like outlier channels, norms over five decades, small and large magnitudes inside the
    fp16 norm's range, mostly-zero rows, one-hot rows; a few all-zero rows in each."""
    x = rng.standard_normal(shape)
    if flavour == "outliers":
        x[..., :4] *= 30.0
    elif flavour == "scales":
        x *= np.exp(rng.uniform(-6, 6, size=shape[:2] + (1,)))
    elif flavour == "tiny":
        x *= 1e-4 if dtype == np.float16 else 1e-12
    elif flavour == "huge":
        x *= 1500.0
    elif flavour == "sparse":
        x *= (rng.random(shape) < 0.05)
    elif flavour == "onehot":
        x[:] = 0
        idx = rng.integers(0, D, size=shape[:2])
        np.put_along_axis(x, idx[..., None], rng.standard_normal(shape[:2] + (1,)) + 3.0, axis=2)
    x[rng.random(shape[:2]) < 0.02] = 0
    if dtype == np.float16:
        x = np.clip(x, -60000, 60000)
    return x.astype(dtype)


@pytest.mark.parametrize("seed", range(6))
def test_sweep_codec_paths(seed):
    """Ten cases per seed over store (bytes against the oracle's layout of the same codes), the fused K+V store,
    append in random chunks, requantisation, the fork interchange at the three block sizes and both load domains."""
    tt = L.torch()
    for case in range(10):
        rng = np.random.default_rng(7000 + 100 * seed + case)
        bits = int(rng.choice([2, 3, 4])); kind = str(rng.choice(["k", "v"]))
        dtype = [np.float16, np.float16, np.float32, np.float64][int(rng.integers(0, 4))]
        n_seqs = int(rng.integers(1, 5))
        tokens = int(rng.choice([rng.integers(1, 200), rng.integers(200, 1500), rng.integers(1500, 4000)]))
        flavour = str(rng.choice(["normal", "outliers", "scales", "tiny", "huge", "sparse", "onehot"]))
        what = ["store", "store_kv", "append", "requant", "fork", "load"][(case + seed) % 6]
        print(f"seed {seed} case {case}: {what} bits={bits} kind={kind} {np.dtype(dtype).name} n_seqs={n_seqs} tokens={tokens} {flavour}",
              flush=True)
        codec = tqa.TurboCodec(bits, seed=int(rng.integers(0, 1000)))
        x = _rows(rng, (n_seqs, tokens, D), dtype, flavour)
        x32 = x.astype(np.float32) if dtype == np.float64 else x
        if what == "store":
            packed = codec.store(x, kind=kind)
            idx, g = codec.unpack_codes(packed, n_seqs, tokens, kind=kind)
            idx, g = np_(idx).reshape(-1, D), np_(g).reshape(-1)
            # rows with few non-zero entries put rotated values on a lattice: ties at boundaries are frequent
            check_codes(codec, x.reshape(-1, D), idx, g, max_band_frac=1e-3 if flavour in ("sparse", "onehot") else 2e-5)
            nb = -(-tokens // 128)
            zero_code = int(np.sum(O.midpoints(codec.centroids) < 0.0))
            ip = np.full((n_seqs, nb * 128, D), zero_code, dtype=np.uint8)
            ip[:, :tokens] = idx.reshape(n_seqs, tokens, D)
            gp = np.zeros((n_seqs, nb * 128), dtype=np.float16)
            gp[:, :tokens] = g.reshape(n_seqs, tokens).astype(np.float16)
            assert np.array_equal(np_(packed), O.layout_pack(ip.reshape(-1, D), gp.reshape(-1), bits, kind))
        elif what == "store_kv":
            vc = tqa.TurboCodec(int(rng.choice([2, 3, 4])), seed=int(rng.integers(0, 1000)))
            v = _rows(rng, (n_seqs, tokens, D), x32.dtype.type, flavour)
            pk, pv = codec.store_kv(vc, x32, v)
            assert tt.equal(pk, codec.store(x32, kind="k")) and tt.equal(pv, vc.store(v, kind="v"))
        elif what == "append":
            cap = tokens + int(rng.integers(0, 300))
            x64 = x.astype(np.float64)
            cache = tt.zeros(tqa.packed_bytes(bits, n_seqs, cap), dtype=tt.uint8, device="cuda")
            pos = 0
            while pos < tokens:
                n_new = int(min(tokens - pos, rng.choice([1, 1, 2, 17, 64, 128, 129, 300, 1000])))
                codec.append(x64[:, pos:pos + n_new], cache, pos, cap, kind=kind)
                pos += n_new
            want = np_(codec.store(x64, kind=kind)).reshape(n_seqs, -1, O.block_bytes(bits))
            got = np_(cache).reshape(n_seqs, -1, O.block_bytes(bits))
            assert np.array_equal(got[:, :want.shape[1]], want) and not got[:, want.shape[1]:].any()
        elif what == "requant":
            sb = max(bits, 3)
            src, dst = tqa.TurboCodec(sb, seed=1), tqa.TurboCodec(int(rng.integers(2, sb)), seed=1)
            TP._check_requant(src, dst, src.store(x32, kind=kind), n_seqs, tokens, kind)
        elif what == "fork":
            bv = 128 if bits == 4 else int(rng.choice([32, 64, 128]))
            packed = codec.store(x32, kind=kind)
            idx, g = codec.unpack_codes(packed, n_seqs, tokens, kind=kind)
            blocks = codec.export_fork_blocks(packed, n_seqs, tokens, kind=kind, block_values=bv)
            want = O.fork_blocks_pack(np_(idx).reshape(-1, D), np_(g).reshape(-1).astype(np.float16), bits, bv)
            assert np.array_equal(np_(blocks).reshape(want.shape), want)
            assert tt.equal(codec.import_fork_blocks(blocks, kind=kind, block_values=bv), packed)
        else:
            packed = codec.store(x32, kind=kind)
            idx, g = codec.unpack_codes(packed, n_seqs, tokens, kind=kind)
            rot = O.turbo_decode_rotated(np_(idx), np_(g).astype(np.float64), codec.centroids)
            got = np_(codec.load(packed, n_seqs, tokens, kind=kind, domain="rotated"))
            assert np.all(np.abs(got - rot) <= 2e-6 * (np.abs(rot).max(axis=-1, keepdims=True) + 1e-300) + 1e-30)
            orig = O.rotate_fast(rot, codec.signs1, codec.signs2, D, transpose=True)
            got = np_(codec.load(packed, n_seqs, tokens, kind=kind, domain="original"))
            assert np.all(np.abs(got - orig) <= 4e-6 * np.linalg.norm(rot, axis=-1, keepdims=True) + 1e-30)


@pytest.mark.parametrize("seed", range(6))
def test_sweep_decode_attention(seed):
    """Ten cases per seed over head sizes, every K x V format pair, groups of 1 to 12 query heads, 1 to 64 splits
    (or the default), Sparse V, dense / sparse / both biases and caches laid out for more tokens than they hold."""
    tt = L.torch()
    for case in range(10):
        rng = np.random.default_rng(9000 + 100 * seed + case)
        hd = int(rng.choice([128, 128, 256]))
        kf, vf = str(rng.choice(["t2", "t3", "t4", "q8"])), str(rng.choice(["t2", "t3", "t4", "q8"]))
        if hd == 256 and kf != "q8" and vf != "q8" and int(kf[1]) < int(vf[1]):
            kf, vf = vf, kf                                      # 256-dim heads: turbo K at least as wide as turbo V
        B, Hkv, G = int(rng.integers(1, 4)), int(rng.integers(1, 4)), int(rng.choice([1, 2, 3, 4, 5, 8, 12]))
        Hq = G * Hkv
        N = int(rng.choice([rng.integers(1, 130), rng.integers(130, 1200), rng.integers(1200, 4000)]))
        ns = int(rng.choice([0, 1, 2, 3, 4, 8, 16, 32, 64]))
        tau = float(rng.choice([0.0, 0.0, 1e-3]))
        bias_kind = str(rng.choice(["none", "none", "dense", "sparse", "both"]))
        cap = 0 if rng.random() < 0.6 or hd == 256 else N + int(rng.integers(0, 300))
        print(f"seed {seed} case {case}: hd={hd} k={kf} v={vf} B={B} Hkv={Hkv} G={G} N={N} splits={ns} tau={tau} bias={bias_kind} cap={cap}",
              flush=True)
        rows = tqa.rows_of_256 if hd == 256 else (lambda t: t)
        Lr = cap if cap else N
        k = rng.standard_normal((B * Hkv, Lr, hd)).astype(np.float16)
        v = rng.standard_normal((B * Hkv, Lr, hd)).astype(np.float16)
        k[:, N:] = 0
        v[:, N:] = 0
        q = (rng.standard_normal((B, Hq, hd)) * rng.choice([1.0, 2.0])).astype(np.float16)
        kc = None if kf == "q8" else tqa.TurboCodec(int(kf[1]), seed=42)
        vc = None if vf == "q8" else tqa.TurboCodec(int(vf[1]), seed=542)
        kp = tqa.q8_0_store(rows(k), kind="k")[0] if kc is None else kc.store(rows(k), kind="k")
        vp = tqa.q8_0_store(rows(v), kind="v")[0] if vc is None else vc.store(rows(v), kind="v")
        kw = dict(head_dim=hd, sparse_v_tau=tau, poison_output=True)
        if ns:
            kw["n_splits"] = ns
        if cap:
            kw["capacity"] = cap
        attn = tqa.DecodeAttention(kc, vc, B, Hq, Hkv, N, **kw)
        bias = bd = sb = None
        if bias_kind != "none":
            bias = np.zeros((B, Hq, N), dtype=np.float32)
            for _ in range(int(rng.integers(1, 6))):
                bias[rng.integers(0, B), rng.integers(0, Hq), rng.integers(0, N)] = float(rng.normal() * 3)
            bias[:, :, : min(3, N)] += 2.0
            bt = tt.from_numpy(bias).cuda()
            if bias_kind == "dense":
                bd = bt
            elif bias_kind == "sparse":
                sb = tqa.sparse_bias_from_dense(bt)
            else:
                bd = bt.clone()
                bd[:, :, N // 2:] = 0
                sb = tqa.sparse_bias_from_dense(bt - bd)
        out = np_(attn(q, kp, vp, bias=bd, sparse_bias=sb)).copy()
        b64 = None if bias is None else bias.astype(np.float64)
        nsp, scale = attn.params.n_splits, 1 / np.sqrt(hd)
        if hd == 256:
            r = TA.reference_attention_256(q, kc, vc, kp, vp, B, Hq, Hkv, N, scale, k_q8=kp if kc is None else None,
                                           v_q8=vp if vc is None else None, n_splits=nsp, tau=tau, bias=b64)
            ref, sk = r if tau > 0 else (r, None)
        else:
            ref, sk, _ = TA.reference_attention(q, kc, vc, kp, vp, B, Hq, Hkv, N, scale, n_splits=nsp, tau=tau, bias=b64,
                                                k_q8=kp if kc is None else None, v_q8=vp if vc is None else None,
                                                capacity=cap if cap else None)
        assert np.isfinite(out).all()
        TA.assert_close(out, ref)
        if tau > 0:
            assert abs(attn.skip_rate() - sk) < 3e-3


@pytest.mark.parametrize("seed", range(3))
def test_sweep_reference_api(seed):
    """Ten cases per seed over the float64 reference-API kernels: any d from 1 to 1024 (odd, padded, power of two),
    1 to 4 bits, dense and WHT rotations, both projection kinds, magnitudes from 1e-9 to 1e9."""
    for case in range(10):
        rng = np.random.default_rng(5000 + 100 * seed + case)
        d = int(rng.choice([1, 2, 3, 5, 8, 17, 32, 64, 96, 100, 128, 129, 200, 256, 384, 512, 777, 1024]))
        b = int(rng.choice([1, 2, 3, 4]))
        n = int(rng.choice([1, 2, 7, 33, 150]))
        rot = str(rng.choice(["dense", "dense", "wht"]))
        what = ["polar", "qjl", "turbo"][(case + seed) % 3]
        s = int(rng.integers(0, 10000))
        scale = float(np.exp(rng.uniform(-20, 20)))
        print(f"seed {seed} case {case}: {what} d={d} b={b} n={n} rot={rot} scale={scale:.3g}", flush=True)
        x = rng.standard_normal((n, d)) * scale
        if n > 2:
            x[1] = 0
        if what == "polar":
            g, o = tqa.PolarQuant(d, b, seed=s, rotation=rot), O.PolarRef(d, b, seed=s, rotation=rot)
            ig, ng = g.quantize(x)
            io, no = o.quantize(x)
            y, _ = o.rotated(x)
            n_bad, n_inadm = O.boundary_band_mismatches(y, ig, o.centroids, rel=1e-11)
            assert n_inadm == 0 and n_bad <= 2, (n_bad, n_inadm)
            np.testing.assert_allclose(ng, no, rtol=1e-13)
            np.testing.assert_allclose(g.dequantize(io, no), o.dequantize(io, no), rtol=1e-9, atol=1e-12 * scale)
        elif what == "qjl":
            mode = str(rng.choice(["orthogonal", "gaussian"]))
            g, o = tqa.QJL(d, seed=s, projection=mode), O.QJLRef(d, seed=s, projection=mode)
            zg, ng = g.quantize(x)
            zo, no = o.quantize(x)
            bad = zg != zo
            assert np.all(np.abs(o.project(x))[bad] <= 1e-11 * np.linalg.norm(x, axis=1).max()) and bad.sum() <= 2
            np.testing.assert_allclose(ng, no, rtol=1e-13)
            np.testing.assert_allclose(g.dequantize(zo, no), o.dequantize(zo, no), rtol=1e-9, atol=1e-12 * scale)
        else:
            b = max(b, 2)
            g, o = tqa.TurboQuant(d, b, seed=s), O.TurboRef(d, b, seed=s)
            co = o.quantize(x)
            np.testing.assert_allclose(g.dequantize(co), o.dequantize(co), rtol=1e-8, atol=1e-11 * scale)
            cg = g.quantize(x)
            same = np.all(cg.mse_indices == co.mse_indices, axis=-1) & np.all(cg.qjl_signs == co.qjl_signs, axis=-1)
            assert same.sum() >= n - 1
            np.testing.assert_allclose(g.dequantize(cg)[same], o.dequantize(co)[same], rtol=1e-8, atol=1e-11 * scale)
