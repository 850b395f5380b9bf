"""GPU parity of attention over packed KV and of the score tile against the
oracle.  The oracle consumes the codes the GPU stored (unpacked through the
C ABI), so these tests isolate the attention arithmetic; the store itself is
checked in test_gpu_turbo.py.

Tolerance: queries, centroid pairs and softmax weights enter the MFMA as fp16
(fp32 accumulation), so outputs are held to the fp16-I/O bar: max abs error
<= 2e-3 * max|reference| per query row."""
import numpy as np
import pytest

import tq_oracle as O
import turboquant_plus_amd as tqa
from turboquant_plus_amd import _lib as L

pytestmark = pytest.mark.gpu
D = 128


def np_(t):
    return t.detach().cpu().numpy()


def reference_attention(q, kc, vc, k_packed, v_packed, B, Hq, Hkv, N, scale, n_splits=1, tau=0.0, bias=None,
                        k_q8=None, v_q8=None, capacity=None):
    """Oracle attention on the GPU-stored codes -> (out [B,Hq,128], skip rate, final-weight rate).
    capacity: the buffers are caches laid out for that many tokens per sequence, of which the first N count."""
    G = Hq // Hkv
    L_ = N if capacity is None else capacity   # tokens per sequence the buffers are laid out for
    if k_q8 is None:
        ki, kg = kc.unpack_codes(k_packed, B * Hkv, L_, kind="k")
        k_rot = O.turbo_decode_rotated(np_(ki)[:, :N], np_(kg)[:, :N].astype(np.float64), kc.centroids)
        q_rot = O.rotate_fast(q.astype(np.float64), kc.signs1, kc.signs2, D)
    else:
        qq, ss = tqa.q8_0_unpack(k_q8, B * Hkv, L_)
        k_rot = O.q8_0_dequantize(np_(qq), np_(ss))[:, :N]
        q_rot = q.astype(np.float64)
    if v_q8 is None:
        vi, vg = vc.unpack_codes(v_packed, B * Hkv, L_, kind="v")
        v_rot = O.turbo_decode_rotated(np_(vi)[:, :N], np_(vg)[:, :N].astype(np.float64), vc.centroids)
    else:  # q8_0-style V: stored unrotated
        qq, ss = tqa.q8_0_unpack(v_q8, B * Hkv, L_, kind="v")
        v_rot = O.q8_0_dequantize(np_(qq), np_(ss))[:, :N]
    out = np.zeros((B, Hq, D))
    skipped = below = 0.0
    for b in range(B):
        for h in range(Hkv):
            g = b * Hkv + h
            qs = q_rot[b, h * G:(h + 1) * G]
            bb = None if bias is None else bias[b, h * G:(h + 1) * G]
            o, sk, fr = O.decode_attention(qs, k_rot[g], v_rot[g], scale, n_splits=n_splits, sparse_v_tau=tau,
                                           logit_bias=bb)
            out[b, h * G:(h + 1) * G] = o if v_q8 is not None else O.rotate_fast(o, vc.signs1, vc.signs2, D, transpose=True)
            skipped += sk
            below += fr
    return out, skipped / (B * Hkv), below / (B * Hkv)


def assert_close(got, ref, rel=2e-3):
    err = np.abs(got - ref).max(axis=-1)
    bound = rel * np.abs(ref).max(axis=-1)
    assert np.all(err <= bound), f"max err/bound = {(err / bound).max():.3f}"


def make_kv(B, Hkv, N, seed, kbits=3, vbits=3):
    rng = np.random.default_rng(seed)
    k = rng.standard_normal((B * Hkv, N, D)).astype(np.float16)
    v = rng.standard_normal((B * Hkv, N, D)).astype(np.float16)
    kc = tqa.TurboCodec(kbits, seed=42)
    vc = tqa.TurboCodec(vbits, seed=542)
    return k, v, kc, vc, kc.store(k, kind="k"), vc.store(v, kind="v")


@pytest.mark.parametrize("N,n_splits", [(64, 1), (128, 1), (100, 1), (1000, 3), (2048, 4), (4096 + 37, 8), (8192, 64),
                                        (8192, 128), (16384, 256)])   # the last two: 32 and 64 partials per group
def test_decode_attention_turbo3(N, n_splits):
    B, Hq, Hkv = 2, 8, 2
    k, v, kc, vc, kp, vp = make_kv(B, Hkv, N, seed=N)
    q = np.random.default_rng(N + 1).standard_normal((B, Hq, D)).astype(np.float16)
    attn = tqa.DecodeAttention(kc, vc, B, Hq, Hkv, N, n_splits=n_splits)
    out = np_(attn(q, kp, vp))
    ref, _, _ = reference_attention(q, kc, vc, kp, vp, B, Hq, Hkv, N, 1 / np.sqrt(D))
    assert_close(out, ref)
    # the split count only moves the running maxima, i.e. the fp16 rounding of the weights
    out1 = np_(tqa.DecodeAttention(kc, vc, B, Hq, Hkv, N, n_splits=1)(q, kp, vp)).copy()
    np.testing.assert_allclose(out, out1, rtol=0, atol=1e-3 * np.abs(ref).max())


@pytest.mark.parametrize("B,N,n_splits,Hq,sparse", [(256, 256, 2, 32, False), (64, 1024, 8, 32, False), (512, 128, 1, 32, False),
                                                     (256, 200, 2, 16, True), (256, 256, 4, 64, False)])
def test_decode_attention_many_short_sequences(B, N, n_splits, Hq, sparse):
    """Short contexts: a group has fewer splits than a workgroup has wavefronts, so several (batch, kv head) groups
    share a workgroup and its decode tables (8, 2 and 16 groups per workgroup here; 2 with eight heads per pass),
    each group merged by its own wavefronts.  Checked on a sample of the groups."""
    Hkv = 8
    tt = L.torch()
    g = tt.Generator(device="cuda").manual_seed(B + N)
    k = tt.randn((B * Hkv, N, D), generator=g, device="cuda").to(tt.float16)
    v = tt.randn((B * Hkv, N, D), generator=g, device="cuda").to(tt.float16)
    q = tt.randn((B, Hq, D), generator=g, device="cuda").to(tt.float16)
    kc, vc = tqa.TurboCodec(3, seed=42), tqa.TurboCodec(3, seed=542)
    kp, vp = kc.store(k, kind="k"), vc.store(v, kind="v")
    tau = 1e-3 if sparse else 0.0
    attn = tqa.DecodeAttention(kc, vc, B, Hq, Hkv, N, n_splits=n_splits, sparse_v_tau=tau)
    out = np_(attn(q, kp, vp))
    # oracle on a few sequences (all their kv heads), from the stored codes
    per = tqa.packed_bytes(3, Hkv, N)
    for b in (0, 1, B // 2 + 1, B - 1):
        ref, sk, _ = reference_attention(np_(q[b:b + 1]), kc, vc, kp[b * per:(b + 1) * per], vp[b * per:(b + 1) * per], 1, Hq, Hkv, N,
                                         1 / np.sqrt(D), n_splits=n_splits, tau=tau)
        assert_close(out[b:b + 1], ref)
    # and every row was written
    assert np.isfinite(out).all()


def reference_attention_256(q, kc, vc, k_packed, v_packed, B, Hq, Hkv, N, scale, k_q8=None, n_splits=1, tau=0.0, bias=None,
                            v_q8=None):
    """Oracle attention for heads of 256 dims on the GPU-stored codes: the caches hold 2 N rows of 128 per sequence,
    row 2 t + half; a token's vector is its two rows side by side, each decoded and un-rotated by itself."""
    G = Hq // Hkv
    if k_q8 is None:
        ki, kg = kc.unpack_codes(k_packed, B * Hkv, 2 * N, kind="k")
        k_rot = O.turbo_decode_rotated(np_(ki), np_(kg).astype(np.float64), kc.centroids).reshape(B * Hkv, N, 2 * D)
        q_rot = O.rotate_fast(q.astype(np.float64).reshape(B, Hq, 2, D), kc.signs1, kc.signs2, D).reshape(B, Hq, 2 * D)
    else:
        qq, ss = tqa.q8_0_unpack(k_q8, B * Hkv, 2 * N)
        k_rot = O.q8_0_dequantize(np_(qq), np_(ss)).reshape(B * Hkv, N, 2 * D)
        q_rot = q.astype(np.float64)
    if v_q8 is None:
        vi, vg = vc.unpack_codes(v_packed, B * Hkv, 2 * N, kind="v")
        v_rot = O.turbo_decode_rotated(np_(vi), np_(vg).astype(np.float64), vc.centroids).reshape(B * Hkv, N, 2 * D)
    else:                                      # q8_0-style V rows: stored unrotated
        qq, ss = tqa.q8_0_unpack(v_q8, B * Hkv, 2 * N, kind="v")
        v_rot = O.q8_0_dequantize(np_(qq), np_(ss)).reshape(B * Hkv, N, 2 * D)
    out = np.zeros((B, Hq, 2 * D))
    skipped = 0.0
    for b in range(B):
        for h in range(Hkv):
            g = b * Hkv + h
            bb = None if bias is None else bias[b, h * G:(h + 1) * G]
            o, sk, _ = O.decode_attention(q_rot[b, h * G:(h + 1) * G], k_rot[g], v_rot[g], scale, n_splits=n_splits,
                                          sparse_v_tau=tau, logit_bias=bb, tile=32)
            if v_q8 is None:
                o = O.rotate_fast(o.reshape(G, 2, D), vc.signs1, vc.signs2, D, transpose=True)
            out[b, h * G:(h + 1) * G] = o.reshape(G, 2 * D)
            skipped += sk
    return (out, skipped / (B * Hkv)) if tau > 0 else out


@pytest.mark.parametrize("bits", [3, 4, 2])
@pytest.mark.parametrize("N,n_splits,Hq", [(32, 1, 8), (64, 1, 8), (100, 1, 8), (1000, 3, 8), (4096 + 37, 8, 8), (2048, 16, 6),
                                           (1536, 32, 16), (77, 2, 2)])
def test_decode_attention_head_dim_256(bits, N, n_splits, Hq):
    """Heads of 256 dims: two 128-value groups per vector, each with its own rotation, codes and norm; the caches are
    those of 128-dim heads with two rows per token.  Groups of 4, 3, 8 (two passes) and 1 query heads per KV head,
    ragged last tiles, one to 32 splits."""
    B, Hkv = 2, 2
    rng = np.random.default_rng(1000 * bits + N)
    k = rng.standard_normal((B * Hkv, N, 2 * D)).astype(np.float16)
    v = rng.standard_normal((B * Hkv, N, 2 * D)).astype(np.float16)
    k[:, :, 128:] *= 2.0                       # the halves have norms of their own
    v[:, :, :128] *= 0.5
    kc, vc = tqa.TurboCodec(bits, seed=42), tqa.TurboCodec(bits, seed=542)
    kp = kc.store(tqa.rows_of_256(k), kind="k")
    vp = vc.store(tqa.rows_of_256(v), kind="v")
    q = rng.standard_normal((B, Hq, 2 * D)).astype(np.float16)
    attn = tqa.DecodeAttention(kc, vc, B, Hq, Hkv, N, n_splits=n_splits, head_dim=256)
    out = np_(attn(q, kp, vp))
    assert out.shape == (B, Hq, 2 * D)
    ref = reference_attention_256(q, kc, vc, kp, vp, B, Hq, Hkv, N, 1 / np.sqrt(2 * D))
    assert_close(out, ref)


@pytest.mark.parametrize("kbits,vbits", [(8, 4), (8, 3), (8, 2), (4, 2), (3, 2), (4, 3), (8, 8), (4, 8), (3, 8), (2, 8)])
@pytest.mark.parametrize("N,n_splits", [(100, 1), (2048 + 31, 8)])
def test_decode_attention_head_dim_256_mixed_formats(kbits, vbits, N, n_splits):
    """256-dim heads with q8_0-style K rows (the fork's recommended "-ctk q8_0 -ctv turboN"), with K wider than V, and
    with q8_0-style V rows (the boundary layers of the fork's Boundary V policy)."""
    B, Hq, Hkv = 2, 8, 2
    rng = np.random.default_rng(100 * kbits + vbits + N)
    k = rng.standard_normal((B * Hkv, N, 2 * D)).astype(np.float16)
    v = rng.standard_normal((B * Hkv, N, 2 * D)).astype(np.float16)
    k[:, :, :7] *= 4.0
    if vbits == 8:
        v[:, :, 128:] *= 3.0                   # the halves' 32-value groups have scales of their own
        v[:, 5::7, 40:72] *= 0.25
        vc, vp = None, tqa.q8_0_store(tqa.rows_of_256(v), kind="v")[0]
    else:
        vc = tqa.TurboCodec(vbits, seed=542)
        vp = vc.store(tqa.rows_of_256(v), kind="v")
    q = rng.standard_normal((B, Hq, 2 * D)).astype(np.float16)
    if kbits == 8:
        kc, kp = None, tqa.q8_0_store(tqa.rows_of_256(k))[0]
    else:
        kc = tqa.TurboCodec(kbits, seed=42)
        kp = kc.store(tqa.rows_of_256(k), kind="k")
    attn = tqa.DecodeAttention(kc, vc, B, Hq, Hkv, N, n_splits=n_splits, head_dim=256)
    out = np_(attn(q, kp, vp))
    ref = reference_attention_256(q, kc, vc, kp, vp, B, Hq, Hkv, N, 1 / np.sqrt(2 * D), k_q8=kp if kbits == 8 else None,
                                  v_q8=vp if vbits == 8 else None)
    assert_close(out, ref)


def test_decode_attention_head_dim_256_grows_by_append():
    """A 256-dim cache that grows in place: prefill and appends work on rows (two per token, positions and capacity
    counted in rows), attention on tokens."""
    B, Hq, Hkv, cap, N0 = 2, 8, 2, 512, 200
    rng = np.random.default_rng(12)
    kc, vc = tqa.TurboCodec(3, seed=42), tqa.TurboCodec(3, seed=542)
    k = rng.standard_normal((B * Hkv, N0 + 3, 2 * D)).astype(np.float16)
    v = rng.standard_normal((B * Hkv, N0 + 3, 2 * D)).astype(np.float16)
    tt = L.torch()
    ck = tt.zeros(tqa.packed_bytes(3, B * Hkv, 2 * cap), dtype=tt.uint8, device="cuda")
    cv = tt.zeros_like(ck)
    kc.append_kv(vc, tqa.rows_of_256(k[:, :N0]), tqa.rows_of_256(v[:, :N0]), ck, cv, 0, 2 * cap)
    attn = tqa.DecodeAttention(kc, vc, B, Hq, Hkv, N0, n_splits=4, capacity=cap, head_dim=256)
    for step in range(3):
        n = N0 + step
        kc.append_kv(vc, tqa.rows_of_256(k[:, n:n + 1]), tqa.rows_of_256(v[:, n:n + 1]), ck, cv, 2 * n, 2 * cap)
        attn.set_tokens(n + 1)
        q = rng.standard_normal((B, Hq, 2 * D)).astype(np.float16)
        out = np_(attn(q, ck, cv)).copy()
        kp = kc.store(tqa.rows_of_256(np.ascontiguousarray(k[:, :n + 1])), kind="k")
        vp = vc.store(tqa.rows_of_256(np.ascontiguousarray(v[:, :n + 1])), kind="v")
        want = np_(tqa.DecodeAttention(kc, vc, B, Hq, Hkv, n + 1, n_splits=4, head_dim=256)(q, kp, vp))
        np.testing.assert_allclose(out, want, rtol=0, atol=2e-3 * np.abs(want).max())


@pytest.mark.parametrize("N,n_splits", [(100, 1), (2048 + 31, 8), (4096, 32)])
def test_decode_attention_head_dim_256_sparse_v_and_bias(N, n_splits):
    """256-dim heads with Sparse V (the skip test runs on tiles of 32 tokens: a token is two rows of a 64-row tile),
    a dense logit bias, a sparse one, and both."""
    B, Hq, Hkv = 2, 8, 2
    rng = np.random.default_rng(N)
    k = rng.standard_normal((B * Hkv, N, 2 * D)).astype(np.float16)
    v = rng.standard_normal((B * Hkv, N, 2 * D)).astype(np.float16)
    kc, vc = tqa.TurboCodec(3, seed=42), tqa.TurboCodec(3, seed=542)
    kp, vp = kc.store(tqa.rows_of_256(k), kind="k"), vc.store(tqa.rows_of_256(v), kind="v")
    q = (2.0 * rng.standard_normal((B, Hq, 2 * D))).astype(np.float16)
    scale = 1 / np.sqrt(2 * D)
    tau = 1e-3
    attn = tqa.DecodeAttention(kc, vc, B, Hq, Hkv, N, n_splits=n_splits, head_dim=256, sparse_v_tau=tau)
    out = np_(attn(q, kp, vp)).copy()
    ref, sk = reference_attention_256(q, kc, vc, kp, vp, B, Hq, Hkv, N, scale, n_splits=n_splits, tau=tau)
    assert_close(out, ref)
    assert abs(attn.skip_rate() - sk) < 2e-3 and sk > 0.05
    bias = np.zeros((B, Hq, N), dtype=np.float32)
    bias[:, :, : min(4, N)] = 3.0
    bias[:, 1::2, N - 1] = -2.0
    bias[0, 0, N // 2] = 5.0
    dense = tqa.DecodeAttention(kc, vc, B, Hq, Hkv, N, n_splits=n_splits, head_dim=256)
    ref_b = reference_attention_256(q, kc, vc, kp, vp, B, Hq, Hkv, N, scale, bias=bias.astype(np.float64))
    bd = L.torch().from_numpy(bias).cuda()
    assert_close(np_(dense(q, kp, vp, bias=bd)), ref_b)
    assert_close(np_(dense(q, kp, vp, sparse_bias=tqa.sparse_bias_from_dense(bd))), ref_b)
    half = bd.clone()
    half[:, :, N // 2:] = 0
    assert_close(np_(dense(q, kp, vp, bias=half, sparse_bias=tqa.sparse_bias_from_dense(bd - half))), ref_b)
    out_sb, sk_b = reference_attention_256(q, kc, vc, kp, vp, B, Hq, Hkv, N, scale, n_splits=n_splits, tau=tau, bias=bias.astype(np.float64))
    assert_close(np_(attn(q, kp, vp, sparse_bias=tqa.sparse_bias_from_dense(bd))), out_sb)


@pytest.mark.parametrize("kbits", [8, 3])
def test_decode_attention_head_dim_256_q8_v_rows_sparse_v_and_bias(kbits):
    """256-dim heads on q8_0-style V rows with Sparse V, a dense and a sparse logit bias, and a group of three query
    heads per KV head (a pass with an idle head row)."""
    B, Hq, Hkv, N, n_splits = 2, 6, 2, 2048 + 31, 8
    rng = np.random.default_rng(77 + kbits)
    k = rng.standard_normal((B * Hkv, N, 2 * D)).astype(np.float16)
    v = rng.standard_normal((B * Hkv, N, 2 * D)).astype(np.float16)
    v[:, :, 128:] *= 2.0
    if kbits == 8:
        kc, kp = None, tqa.q8_0_store(tqa.rows_of_256(k))[0]
    else:
        kc = tqa.TurboCodec(kbits, seed=42)
        kp = kc.store(tqa.rows_of_256(k), kind="k")
    vp = tqa.q8_0_store(tqa.rows_of_256(v), kind="v")[0]
    q = (2.0 * rng.standard_normal((B, Hq, 2 * D))).astype(np.float16)
    scale, tau = 1 / np.sqrt(2 * D), 1e-3
    kq = kp if kbits == 8 else None
    attn = tqa.DecodeAttention(kc, None, B, Hq, Hkv, N, n_splits=n_splits, head_dim=256, sparse_v_tau=tau)
    out = np_(attn(q, kp, vp)).copy()
    ref, sk = reference_attention_256(q, kc, None, kp, vp, B, Hq, Hkv, N, scale, k_q8=kq, v_q8=vp, n_splits=n_splits, tau=tau)
    assert_close(out, ref)
    assert abs(attn.skip_rate() - sk) < 2e-3 and sk > 0.05
    bias = np.zeros((B, Hq, N), dtype=np.float32)
    bias[:, :, :4] = 3.0
    bias[:, 1::2, N - 1] = -2.0
    bias[0, 0, N // 2] = 5.0
    bd = L.torch().from_numpy(bias).cuda()
    dense = tqa.DecodeAttention(kc, None, B, Hq, Hkv, N, n_splits=n_splits, head_dim=256)
    ref_b = reference_attention_256(q, kc, None, kp, vp, B, Hq, Hkv, N, scale, k_q8=kq, v_q8=vp, bias=bias.astype(np.float64))
    assert_close(np_(dense(q, kp, vp, bias=bd)), ref_b)
    assert_close(np_(dense(q, kp, vp, sparse_bias=tqa.sparse_bias_from_dense(bd))), ref_b)


def test_decode_attention_head_dim_256_refuses_what_it_does_not_take():
    B, Hq, Hkv, N = 1, 4, 1, 128
    kc, vc = tqa.TurboCodec(3, seed=42), tqa.TurboCodec(3, seed=542)
    tt = L.torch()
    buf = tt.zeros(tqa.packed_bytes(3, B * Hkv, 2 * N), dtype=tt.uint8, device="cuda")
    q = tt.zeros((B, Hq, 256), dtype=tt.float16, device="cuda")
    with pytest.raises(NotImplementedError):
        tqa.DecodeAttention(tqa.TurboCodec(2, seed=42), vc, B, Hq, Hkv, N, head_dim=256)(q, buf, buf)   # K narrower than V
    with pytest.raises(ValueError):
        tqa.DecodeAttention(kc, vc, B, Hq, Hkv, N, head_dim=64)


@pytest.mark.parametrize("bits", [2, 3, 4])
@pytest.mark.parametrize("n_splits", [16, 3])
def test_decode_attention_with_unequal_codebooks_of_one_width(bits, n_splits):
    """K and V of the same width with different centroids cannot share a decode table: both tables and the
    workgroup's merge space are in LDS at once."""
    B, Hq, Hkv, N = 2, 8, 2, 2048 + 64
    rng = np.random.default_rng(bits + n_splits)
    k = rng.standard_normal((B * Hkv, N, D)).astype(np.float16)
    v = rng.standard_normal((B * Hkv, N, D)).astype(np.float16)
    kc = tqa.TurboCodec(bits, seed=42, centroids=tqa.PRODUCTION_CENTROIDS[bits])
    vc = tqa.TurboCodec(bits, seed=542)
    kp, vp = kc.store(k, kind="k"), vc.store(v, kind="v")
    q = rng.standard_normal((B, Hq, D)).astype(np.float16)
    for tau in (0.0, 1e-4):
        attn = tqa.DecodeAttention(kc, vc, B, Hq, Hkv, N, n_splits=n_splits, sparse_v_tau=tau)
        out = np_(attn(q, kp, vp))
        ref, _, _ = reference_attention(q, kc, vc, kp, vp, B, Hq, Hkv, N, 1 / np.sqrt(D), n_splits=n_splits, tau=tau)
        assert_close(out, ref)


@pytest.mark.parametrize("B,Hkv,N,n_splits,capacity", [
    (1, 1, 64, 32, 0),        # one tile, 31 empty splits in a 16-wavefront workgroup
    (1, 2, 200, 16, 0),       # 4 tiles over 16 splits: 12 empty, last tile ragged
    (3, 1, 1000, 48, 1024),   # 48 = 3 workgroups of 16 splits; cache laid out for 1024 tokens
    (2, 2, 1537, 32, 2048),   # ragged tail, capacity stride
    (1, 3, 4000, 6, 0),       # 6 splits: workgroups of 2 wavefronts
    (5, 1, 777, 7, 0),        # odd split count: one wavefront per workgroup
])
def test_decode_attention_split_and_capacity_shapes(B, Hkv, N, n_splits, capacity):
    Hq = 4 * Hkv
    rng = np.random.default_rng(N + n_splits)
    cap = capacity or N
    k = rng.standard_normal((B * Hkv, N, D)).astype(np.float16)
    v = rng.standard_normal((B * Hkv, N, D)).astype(np.float16)
    kc, vc = tqa.TurboCodec(3, seed=42), tqa.TurboCodec(3, seed=542)
    tt = L.torch()
    ck = tt.zeros(tqa.packed_bytes(3, B * Hkv, cap), dtype=tt.uint8, device="cuda")
    cv = tt.zeros_like(ck)
    kc.append_kv(vc, k, v, ck, cv, 0, cap)
    q = rng.standard_normal((B, Hq, D)).astype(np.float32)
    out = np_(tqa.DecodeAttention(kc, vc, B, Hq, Hkv, N, n_splits=n_splits, capacity=capacity)(q, ck, cv))
    kp, vp = kc.store(k, kind="k"), vc.store(v, kind="v")      # same codes without the capacity stride
    ref, _, _ = reference_attention(q, kc, vc, kp, vp, B, Hq, Hkv, N, 1 / np.sqrt(D))
    assert np.isfinite(out).all()
    assert_close(out, ref)


@pytest.mark.parametrize("kbits,vbits", [(4, 4), (2, 2), (4, 2), (3, 2)])
def test_decode_attention_other_bit_widths(kbits, vbits):
    B, Hq, Hkv, N = 1, 8, 2, 640
    k, v, kc, vc, kp, vp = make_kv(B, Hkv, N, seed=kbits * 10 + vbits, kbits=kbits, vbits=vbits)
    q = np.random.default_rng(5).standard_normal((B, Hq, D)).astype(np.float32)
    out = np_(tqa.DecodeAttention(kc, vc, B, Hq, Hkv, N, n_splits=2)(q, kp, vp))
    ref, _, _ = reference_attention(q, kc, vc, kp, vp, B, Hq, Hkv, N, 1 / np.sqrt(D))
    assert_close(out, ref)


def test_decode_attention_closed_forms():
    """Identical keys -> uniform weights -> mean of V; one dominant key -> its V row."""
    tt = L.torch()
    B, Hq, Hkv, N = 1, 4, 1, 512
    rng = np.random.default_rng(0)
    kc, vc = tqa.TurboCodec(3, seed=42), tqa.TurboCodec(3, seed=542)
    v = rng.standard_normal((1, N, D)).astype(np.float32)
    vp = vc.store(v, kind="v")
    v_hat = np_(vc.load(vp, 1, N, kind="v", domain="original"))[0].astype(np.float64)
    q = rng.standard_normal((B, Hq, D)).astype(np.float32)
    k = np.tile(rng.standard_normal((1, 1, D)).astype(np.float32), (1, N, 1))
    out = np_(tqa.DecodeAttention(kc, vc, B, Hq, Hkv, N, n_splits=2)(q, kc.store(k, kind="k"), vp))
    assert_close(out[0], np.tile(v_hat.mean(0), (4, 1)), rel=3e-3)
    k = (rng.standard_normal((1, N, D)) * 1e-3).astype(np.float32)
    k[0, 300] = 40 * q[0, 2] / np.linalg.norm(q[0, 2])
    out = np_(tqa.DecodeAttention(kc, vc, B, Hq, Hkv, N, n_splits=2)(q, kc.store(k, kind="k"), vp))
    assert_close(out[0, 2:3], v_hat[300:301], rel=3e-3)
    assert tt.isfinite(tt.from_numpy(out)).all()


def test_decode_attention_bias_and_sparse_v():
    B, Hq, Hkv, N = 2, 8, 2, 4096
    k, v, kc, vc, kp, vp = make_kv(B, Hkv, N, seed=77)
    rng = np.random.default_rng(78)
    q = rng.standard_normal((B, Hq, D)).astype(np.float16)
    bias = np.zeros((B, Hq, N), dtype=np.float32)
    for b in range(B):
        for h in range(Hq):
            bias[b, h, rng.choice(N, size=16, replace=False)] = 6.0
    tt = L.torch()
    bias_d = tt.from_numpy(bias).cuda()
    dense = tqa.DecodeAttention(kc, vc, B, Hq, Hkv, N, n_splits=4)
    out_d = np_(dense(q, kp, vp, bias=bias_d)).copy()
    ref_d, _, _ = reference_attention(q, kc, vc, kp, vp, B, Hq, Hkv, N, 1 / np.sqrt(D), bias=bias)
    assert_close(out_d, ref_d)
    for tau in (1e-6, 1e-3):
        sparse = tqa.DecodeAttention(kc, vc, B, Hq, Hkv, N, n_splits=4, sparse_v_tau=tau)
        out_s = np_(sparse(q, kp, vp, bias=bias_d)).copy()
        ref_s, skip_o, below_o = reference_attention(q, kc, vc, kp, vp, B, Hq, Hkv, N, 1 / np.sqrt(D), n_splits=4,
                                                     tau=tau, bias=bias)
        assert_close(out_s, ref_s)
        rate = sparse.skip_rate()
        # the kernel's predicate equals the oracle's up to fp16 logit error near the threshold
        assert abs(rate - skip_o) <= 0.02 * max(skip_o, 1e-3) + 1e-4, (rate, skip_o)
        assert rate <= below_o + 1e-4     # in-kernel test is never looser than the final-weight test
        print(f"\nsparse V tau={tau}: kernel skip rate {rate:.4f}, oracle {skip_o:.4f}, final-weight rate {below_o:.4f}")
        if tau == 1e-6:
            np.testing.assert_allclose(out_s, out_d, rtol=0, atol=1e-4 * np.abs(ref_d).max())


@pytest.mark.parametrize("G,n_splits,N,E", [(4, 4, 1000, 5), (4, 16, 4096, 64), (8, 8, 2111, 70), (1, 1, 64, 3), (6, 32, 2048, 130)])
def test_decode_attention_sparse_bias(G, n_splits, N, E):
    """A logit bias given as per-head (position, value) lists equals the same bias given as dense rows (to rounding: the
    two forms run different instantiations of the kernel, and one adds the scaled bias with a fused multiply-add), and
    both meet the oracle; lists of unequal length (padded), entries at a
    tile's first and last position and at the context's last token, dense and sparse together, Sparse V on top."""
    tt = L.torch()
    B, Hkv = 2, 2
    Hq = Hkv * G
    k, v, kc, vc, kp, vp = make_kv(B, Hkv, N, seed=300 + G)
    rng = np.random.default_rng(E)
    q = rng.standard_normal((B, Hq, D)).astype(np.float16)
    bias = np.zeros((B, Hq, N), dtype=np.float32)
    for b in range(B):
        for h in range(Hq):
            n_e = E if (b + h) % 3 else max(1, E // 2)                   # lists of unequal length
            pos = rng.choice(N, size=min(n_e, N), replace=False)
            bias[b, h, pos] = rng.uniform(2.0, 6.0, size=len(pos)).astype(np.float32)
    bias[0, 0, [0, 63, min(64, N - 1), N - 1]] = [6.0, 5.0, 4.0, 3.0]     # tile edges and the last token
    pos_d, val_d = tqa.sparse_bias_from_dense(bias)
    assert pos_d.shape[2] >= 1 and int((val_d != 0).sum()) == int((bias != 0).sum())
    attn = tqa.DecodeAttention(kc, vc, B, Hq, Hkv, N, n_splits=n_splits)
    dense = np_(attn(q, kp, vp, bias=tt.from_numpy(bias).cuda())).copy()
    sparse = np_(attn(q, kp, vp, sparse_bias=(pos_d, val_d))).copy()
    np.testing.assert_allclose(sparse, dense, rtol=0, atol=2e-6 * np.abs(dense).max())
    ref, _, _ = reference_attention(q, kc, vc, kp, vp, B, Hq, Hkv, N, 1 / np.sqrt(D), n_splits=n_splits, bias=bias)
    assert_close(sparse, ref)
    assert np.abs(sparse - np_(attn(q, kp, vp))).max() > 1e-3            # the bias is not a no-op
    # half of the bias dense, half sparse: they add up
    half = bias * (rng.random(bias.shape) < 0.5)
    p2, v2 = tqa.sparse_bias_from_dense(bias - half)
    both = np_(attn(q, kp, vp, bias=tt.from_numpy(half.astype(np.float32)).cuda(), sparse_bias=(p2, v2)))
    assert_close(both, ref)
    # with Sparse V: the same skipped pairs as with the dense form
    tau = 1e-3
    sv = tqa.DecodeAttention(kc, vc, B, Hq, Hkv, N, n_splits=n_splits, sparse_v_tau=tau)
    a1 = np_(sv(q, kp, vp, bias=tt.from_numpy(bias).cuda())).copy()
    r1 = sv.skip_rate()
    a2 = np_(sv(q, kp, vp, sparse_bias=(pos_d, val_d))).copy()
    np.testing.assert_allclose(a2, a1, rtol=0, atol=2e-6 * np.abs(a1).max())
    assert abs(sv.skip_rate() - r1) <= 1e-5
    with pytest.raises(ValueError):
        attn(q, kp, vp, sparse_bias=(pos_d.to(tt.int64), val_d))


@pytest.mark.parametrize("where", ["front", "back", "spread", "mixed"])
@pytest.mark.parametrize("G,n_splits,head_dim", [(4, 8, 128), (8, 3, 128), (4, 16, 256)])
def test_decode_attention_sparse_bias_long_lists(where, G, n_splits, head_dim):
    """Lists of hundreds of positions per head - runs of consecutive positions at the front or the back of the context
    (a window of recent tokens), every fourth position, and heads with lists of very different lengths: the walk takes
    a head's list sixteen entries at a time, several windows inside one tile and windows that straddle tiles and
    splits.  Equal to the same bias as dense rows, and to the oracle."""
    tt = L.torch()
    B, Hkv, N = 2, 2, 1500
    Hq = Hkv * G
    rng = np.random.default_rng(len(where) + G + head_dim)
    bias = np.zeros((B, Hq, N), dtype=np.float32)
    vals = lambda n: rng.uniform(-3.0, 3.0, size=n).astype(np.float32) + 0.01
    for b in range(B):
        for h in range(Hq):
            if where == "front":
                n_e = 520 if h % 2 else 33
                bias[b, h, :n_e] = vals(n_e)
            elif where == "back":
                n_e = 300 + 17 * h
                bias[b, h, N - n_e:] = vals(n_e)
            elif where == "spread":
                sel = np.arange(h % 4, N, 4)
                bias[b, h, sel] = vals(len(sel))
            else:
                if h % 3 == 0:
                    bias[b, h, 5] = 4.0                                   # one entry
                elif h % 3 == 1:
                    bias[b, h, :] = vals(N)                               # every position
                else:
                    sel = rng.choice(N, size=160, replace=False)
                    bias[b, h, sel] = vals(160)
    pos_d, val_d = tqa.sparse_bias_from_dense(bias)
    bd = tt.from_numpy(bias).cuda()
    if head_dim == 256:
        k = rng.standard_normal((B * Hkv, N, 2 * D)).astype(np.float16)
        v = rng.standard_normal((B * Hkv, N, 2 * D)).astype(np.float16)
        kc, vc = tqa.TurboCodec(3, seed=42), tqa.TurboCodec(3, seed=542)
        kp, vp = kc.store(tqa.rows_of_256(k), kind="k"), vc.store(tqa.rows_of_256(v), kind="v")
        q = rng.standard_normal((B, Hq, 2 * D)).astype(np.float16)
        ref = reference_attention_256(q, kc, vc, kp, vp, B, Hq, Hkv, N, 1 / np.sqrt(2 * D), bias=bias.astype(np.float64))
    else:
        k, v, kc, vc, kp, vp = make_kv(B, Hkv, N, seed=77 + G)
        q = rng.standard_normal((B, Hq, D)).astype(np.float16)
        ref, _, _ = reference_attention(q, kc, vc, kp, vp, B, Hq, Hkv, N, 1 / np.sqrt(D), n_splits=n_splits, bias=bias)
    attn = tqa.DecodeAttention(kc, vc, B, Hq, Hkv, N, n_splits=n_splits, head_dim=head_dim, poison_output=True)
    dense = np_(attn(q, kp, vp, bias=bd)).copy()
    sparse = np_(attn(q, kp, vp, sparse_bias=(pos_d, val_d))).copy()
    # (the two forms add the scaled bias in different instantiations, one with a fused multiply-add: an ulp of a logit, 1e-5 of an output)
    np.testing.assert_allclose(sparse, dense, rtol=0, atol=5e-5 * np.abs(dense).max())
    assert_close(sparse, ref)


@pytest.mark.parametrize("N,misalign", [(1000, 0), (1001, 0), (999, 0), (1000, 1), (64, 0), (67, 1)])
def test_decode_attention_dense_bias_every_position(N, misalign):
    """A bias that differs at every position, for context lengths that are and are not multiples of four and
    for a bias buffer that is not 16-byte aligned: the 16-byte and the element-wise reads give the same."""
    B, Hq, Hkv = 2, 8, 2
    k, v, kc, vc, kp, vp = make_kv(B, Hkv, N, seed=N + misalign)
    rng = np.random.default_rng(N)
    q = rng.standard_normal((B, Hq, D)).astype(np.float16)
    bias = (2.0 * rng.standard_normal((B, Hq, N))).astype(np.float32)
    tt = L.torch()
    buf = tt.zeros(B * Hq * N + 4, dtype=tt.float32, device="cuda")
    bias_d = buf[misalign:misalign + B * Hq * N].view(B, Hq, N)
    bias_d.copy_(tt.from_numpy(bias))
    for n_splits in (1, 3):
        out = np_(tqa.DecodeAttention(kc, vc, B, Hq, Hkv, N, n_splits=n_splits)(q, kp, vp, bias=bias_d))
        ref, _, _ = reference_attention(q, kc, vc, kp, vp, B, Hq, Hkv, N, 1 / np.sqrt(D), n_splits=n_splits, bias=bias)
        assert_close(out, ref)


def test_decode_attention_masked_prefix():
    """-inf bias over a prefix: whole tiles and one whole split carry no weight; output stays finite and equals
    attention over the remaining positions."""
    B, Hq, Hkv, N = 1, 8, 2, 1024
    k, v, kc, vc, kp, vp = make_kv(B, Hkv, N, seed=91)
    q = np.random.default_rng(92).standard_normal((B, Hq, D)).astype(np.float16)
    bias = np.zeros((B, Hq, N), dtype=np.float32)
    bias[:, :, :300] = -np.inf          # split 0 of 4 (tokens 0..255) is masked completely
    bias[:, 3, 300:700] = -np.inf       # one head loses two more splits' worth of tiles
    tt = L.torch()
    out = np_(tqa.DecodeAttention(kc, vc, B, Hq, Hkv, N, n_splits=4)(q, kp, vp, bias=tt.from_numpy(bias).cuda()))
    assert np.isfinite(out).all()
    finite = np.where(np.isfinite(bias), bias, -1e30).astype(np.float32)   # same weights, no inf arithmetic in the oracle
    ref, _, _ = reference_attention(q, kc, vc, kp, vp, B, Hq, Hkv, N, 1 / np.sqrt(D), bias=finite)
    assert_close(out, ref)


def test_decode_attention_many_groups_and_repeated_calls():
    """Thousands of GQA groups with a short context against the oracle (spot-checked groups), and the same call
    repeated many times on one workspace with identical results."""
    B, Hq, Hkv, N = 4100, 4, 1, 128
    k, v, kc, vc, kp, vp = make_kv(B, Hkv, N, seed=93)
    q = np.random.default_rng(94).standard_normal((B, Hq, D)).astype(np.float16)
    out = np_(tqa.DecodeAttention(kc, vc, B, Hq, Hkv, N, n_splits=2)(q, kp, vp))
    sel = [0, 1, 2047, 4095, 4096, 4099]
    ki, kg = kc.unpack_codes(kp, B, N, kind="k")
    vi, vg = vc.unpack_codes(vp, B, N, kind="v")
    k_rot = O.turbo_decode_rotated(np_(ki)[sel], np_(kg)[sel].astype(np.float64), kc.centroids)
    v_rot = O.turbo_decode_rotated(np_(vi)[sel], np_(vg)[sel].astype(np.float64), vc.centroids)
    q_rot = O.rotate_fast(q[sel].astype(np.float64), kc.signs1, kc.signs2, D)
    for n, b in enumerate(sel):
        o, _, _ = O.decode_attention(q_rot[n], k_rot[n], v_rot[n], 1 / np.sqrt(D))
        assert_close(out[b], O.rotate_fast(o, vc.signs1, vc.signs2, D, transpose=True))
    B, Hq, Hkv, N = 2, 8, 2, 1000
    k, v, kc, vc, kp, vp = make_kv(B, Hkv, N, seed=95)
    q = np.random.default_rng(96).standard_normal((B, Hq, D)).astype(np.float16)
    attn = tqa.DecodeAttention(kc, vc, B, Hq, Hkv, N, n_splits=5)
    first = np_(attn(q, kp, vp)).copy()
    ref, _, _ = reference_attention(q, kc, vc, kp, vp, B, Hq, Hkv, N, 1 / np.sqrt(D))
    assert_close(first, ref)
    for _ in range(20):
        again = np_(attn(q, kp, vp))
        assert np.array_equal(again, first)


@pytest.mark.parametrize("n_splits,sparse", [(32, False), (64, False), (32, True)])
def test_in_launch_merge_never_leaves_a_row_unwritten(n_splits, sparse):
    """The split partials of a group are merged inside the launch by the workgroup whose increment completes the group's
    arrival counter.  Shape of the headline step in small: 32 splits = two workgroups of sixteen wavefronts per group (64: four).
    1000 steps back to back on one workspace, the output rows filled with NaN before each: every step must equal the
    first, which is checked against the oracle - a step whose merge found no taker would leave NaN, a merge that ran on
    stale partials would differ.  The Sparse-V total travels through tagged slots of the same workspace and must be the
    first step's too."""
    tt = L.torch()
    B, Hq, Hkv, N = 4, 8, 2, 64 * n_splits
    k, v, kc, vc, kp, vp = make_kv(B, Hkv, N, seed=n_splits)
    q = tt.from_numpy(np.random.default_rng(7).standard_normal((B, Hq, D)).astype(np.float16)).cuda()
    tau = 1e-3 if sparse else 0.0
    attn = tqa.DecodeAttention(kc, vc, B, Hq, Hkv, N, n_splits=n_splits, sparse_v_tau=tau, poison_output=True)
    first = attn(q, kp, vp).clone()
    skip0 = attn.skip.clone()
    ref, sk, _ = reference_attention(np_(q), kc, vc, kp, vp, B, Hq, Hkv, N, 1 / np.sqrt(D), n_splits=n_splits, tau=tau)
    assert_close(np_(first), ref)
    if sparse:
        assert abs(attn.skip_rate() - sk) < 1e-3
    bad = tt.zeros(1, dtype=tt.int64, device="cuda")
    for step in range(1000):
        out = attn(q, kp, vp)
        bad += (~tt.eq(out, first)).sum() + (0 if not sparse else (~tt.eq(attn.skip, skip0)).sum())
        if step % 100 == 99:                 # stop at the first failure, to the nearest hundred steps
            assert int(bad.item()) == 0, f"a step among {step - 99}..{step} left a row unwritten or different"


def test_decode_attention_q8_0_k_turbo2_v():
    """BASELINE config 4 shape family: K q8_0-style (not rotated), V turbo2."""
    B, Hq, Hkv, N = 1, 8, 2, 2048 + 64
    rng = np.random.default_rng(4)
    k = rng.standard_normal((B * Hkv, N, D)).astype(np.float16)
    v = rng.standard_normal((B * Hkv, N, D)).astype(np.float16)
    q = rng.standard_normal((B, Hq, D)).astype(np.float16)
    vc = tqa.TurboCodec(2, seed=542)
    kq, _, _ = tqa.q8_0_store(k)
    vp = vc.store(v, kind="v")
    for tau in (0.0, 1e-6):
        attn = tqa.DecodeAttention(None, vc, B, Hq, Hkv, N, n_splits=3, sparse_v_tau=tau)
        out = np_(attn(q, kq, vp))
        ref, skip_o, _ = reference_attention(q, None, vc, None, vp, B, Hq, Hkv, N, 1 / np.sqrt(D), n_splits=3, tau=tau,
                                             k_q8=kq)
        assert_close(out, ref)
        if tau:
            assert abs(attn.skip_rate() - skip_o) <= 0.02 * max(skip_o, 1e-3) + 1e-4


@pytest.mark.parametrize("kbits,N,n_splits,G", [(None, 2048 + 64, 3, 4), (None, 1000, 16, 4), (3, 1500, 8, 4),
                                                (4, 777, 1, 4), (None, 4096, 32, 2), (3, 300, 2, 6)])
def test_decode_attention_q8_0_v(kbits, N, n_splits, G):
    """V kept as q8_0-style rows (the boundary layers of a layer-adaptive policy), K q8_0-style or turbo.
    The values differ a lot from block to block so that a scale taken from the wrong 32-dim block or the wrong
    token shows."""
    B, Hkv = 2, 2
    Hq = G * Hkv
    rng = np.random.default_rng(1000 + N)
    k = rng.standard_normal((B * Hkv, N, D)).astype(np.float16)
    v = (rng.standard_normal((B * Hkv, N, D)) * np.repeat([0.05, 1.0, 7.0, 0.4], 32) *
         np.exp(rng.standard_normal((B * Hkv, N, 1)))).astype(np.float16)
    q = rng.standard_normal((B, Hq, D)).astype(np.float16)
    kc = tqa.TurboCodec(kbits, seed=42) if kbits else None
    kp = kc.store(k, kind="k") if kbits else tqa.q8_0_store(k)[0]
    vq, _, _ = tqa.q8_0_store(v, kind="v")
    for tau in (0.0, 1e-3):
        attn = tqa.DecodeAttention(kc, None, B, Hq, Hkv, N, n_splits=n_splits, sparse_v_tau=tau)
        out = np_(attn(q, kp, vq))
        ref, skip_o, _ = reference_attention(q, kc, None, kp, None, B, Hq, Hkv, N, 1 / np.sqrt(D), n_splits=n_splits, tau=tau,
                                             k_q8=None if kbits else kp, v_q8=vq)
        assert_close(out, ref)
        if tau:
            assert abs(attn.skip_rate() - skip_o) <= 0.02 * max(skip_o, 1e-3) + 1e-4
    # against the exact values: int8 rows keep V to about 1 % of each 32-value block's largest entry
    if not kbits:
        vt = tqa.TurboCodec(4, seed=542)
        out_t = np_(tqa.DecodeAttention(None, vt, B, Hq, Hkv, N, n_splits=n_splits)(q, kp, vt.store(v, kind="v"))).copy()
        qq, ss = tqa.q8_0_unpack(kp, B * Hkv, N)
        k_hat = O.q8_0_dequantize(np_(qq), np_(ss))
        exact = np.zeros((B, Hq, D))
        for b in range(B):
            for h in range(Hq):
                g = b * Hkv + h // G
                w = O.softmax_rows((q[b, h].astype(np.float64) @ k_hat[g].T / np.sqrt(D))[None])[0]
                exact[b, h] = w @ v[g].astype(np.float64)
        out8 = np_(tqa.DecodeAttention(None, None, B, Hq, Hkv, N, n_splits=n_splits)(q, kp, vq))
        assert np.abs(out8 - exact).max() < 0.25 * np.abs(out_t - exact).max()


def test_decode_attention_rejects_ragged_group():
    kc, vc = tqa.TurboCodec(3), tqa.TurboCodec(3)
    with pytest.raises(ValueError, match="multiple of the KV head count"):
        tqa.DecodeAttention(kc, vc, 1, 7, 2, 128)


@pytest.mark.parametrize("G,n_splits", [(1, 3), (2, 16), (3, 1), (5, 3), (7, 16), (8, 4), (8, 32), (12, 64), (16, 8), (17, 2)])
def test_decode_attention_other_group_sizes(G, n_splits):
    """Query-head groups other than four: up to four heads take one pass of four over the K/V, more take passes of
    eight (two sets of four against the same dequantised rows), short last pass included, with a logit bias per
    (head, position) and the Sparse V count summed over the passes."""
    B, Hkv, N = 2, 3, 1500
    Hq = G * Hkv
    k, v, kc, vc, kp, vp = make_kv(B, Hkv, N, seed=900 + G)
    rng = np.random.default_rng(901 + G)
    q = rng.standard_normal((B, Hq, D)).astype(np.float16)
    bias = (0.5 * rng.standard_normal((B, Hq, N))).astype(np.float32)
    bias_d = L.torch().from_numpy(bias).cuda()
    attn = tqa.DecodeAttention(kc, vc, B, Hq, Hkv, N, n_splits=n_splits)
    out = np_(attn(q, kp, vp, bias=bias_d)).copy()
    ref, _, _ = reference_attention(q, kc, vc, kp, vp, B, Hq, Hkv, N, 1 / np.sqrt(D), bias=bias)
    assert_close(out, ref)
    # every head of a group against the same head served alone (G = 1 layout, same K/V): a head's arithmetic does
    # not depend on which row of the MFMA block it sits in, so the results are bitwise equal when the splits are
    # merged in the same order (groups of up to four heads: workgroups of up to 16 wavefronts, as for one head);
    # groups of more than four heads run eight heads per pass in workgroups of up to 8 wavefronts, which merges
    # 16 or more splits in another order
    for h in (0, G - 1):
        sel = [kv * G + h for kv in range(Hkv)]
        one = tqa.DecodeAttention(kc, vc, B, Hkv, Hkv, N, n_splits=n_splits)
        got = np_(one(np.ascontiguousarray(q[:, sel]), kp, vp, bias=L.torch().from_numpy(np.ascontiguousarray(bias[:, sel])).cuda()))
        if G <= 4 or n_splits < 16:
            assert np.array_equal(got, out[:, sel])
        else:
            np.testing.assert_allclose(got, out[:, sel], rtol=0, atol=2e-6 * np.abs(got).max())
    tau = 1e-3
    sparse = tqa.DecodeAttention(kc, vc, B, Hq, Hkv, N, n_splits=n_splits, sparse_v_tau=tau)
    out_s = np_(sparse(q, kp, vp, bias=bias_d)).copy()
    ref_s, skip_o, _ = reference_attention(q, kc, vc, kp, vp, B, Hq, Hkv, N, 1 / np.sqrt(D), n_splits=n_splits, tau=tau,
                                           bias=bias)
    assert_close(out_s, ref_s)
    rate = sparse.skip_rate()
    assert abs(rate - skip_o) <= 0.02 * max(skip_o, 1e-3) + 1e-4, (rate, skip_o)
    assert int(sparse.skip.cpu()[1]) == B * Hq * N
    # a second call gives the same count (the passes add to a count that the first pass resets)
    sparse(q, kp, vp, bias=bias_d)
    assert sparse.skip_rate() == rate


@pytest.mark.parametrize("projection,nk,nq", [("orthogonal", 1000, 200), ("gaussian", 1000, 200),
                                              ("orthogonal", 333, 70), ("orthogonal", 2304, 513)])
def test_score_tile(projection, nk, nq):
    """TurboQuant inner-product estimator (BASELINE config 5 family, reduced):
    GPU logits against the oracle's on the stored codes, and the estimator's
    bias against the exact inner products."""
    tt = L.torch()
    rng = np.random.default_rng(12)
    keys = rng.standard_normal((nk, D)).astype(np.float32)
    qs = rng.standard_normal((nq, D)).astype(np.float16)
    codec = tqa.TurboCodec(3, seed=42, projection=projection, projection_seed=2)
    packed, sbits, rn = codec.store_qjl(keys)
    logits = np_(codec.score_tile(qs, packed, sbits, rn, nk))
    idx, g = codec.unpack_codes(packed, 1, nk)
    z = np.unpackbits(np_(sbits), axis=1, bitorder="little")[:, :D].astype(np.float64) * 2 - 1
    ref = O.score_tile(qs.astype(np.float64), np_(idx)[0], np_(g)[0].astype(np.float64), codec.centroids,
                       lambda a: O.rotate_fast(a, codec.signs1, codec.signs2, D), codec.S, z,
                       np_(rn).astype(np.float64), codec.projection_scale)
    scale = np.linalg.norm(qs.astype(np.float64), axis=1)[:, None] * np.linalg.norm(keys.astype(np.float64), axis=1)[None, :]
    assert np.abs(logits - ref).max() <= 2e-3 * scale.max() / np.sqrt(D) * 4
    exact = qs.astype(np.float64) @ keys.astype(np.float64).T
    err = logits - exact
    assert abs(err.mean()) < 4 * err.std() / np.sqrt(err.size) + 1e-3       # unbiased
    h = np_(codec.score_tile(qs, packed, sbits, rn, nk, out_dtype=tt.float16)).astype(np.float64)
    assert np.abs(h - ref).max() <= 4e-3 * np.abs(ref).max()


@pytest.mark.parametrize("nk,nq", [(1, 1), (31, 33), (32, 64), (33, 31), (63, 127), (65, 129), (127, 95), (129, 97),
                                   (191, 160), (193, 255), (255, 65), (257, 1), (510, 130), (769, 513)])
def test_score_tile_edges(nk, nq):
    """Row and key edges of the estimator tile: key counts around the 32-key half, the 64-key group of a wavefront
    and the 256-key workgroup, odd ones among them; query counts around the 32-row block, the 64-row half and the
    128-query tile.  Everything outside [nq, nk] must stay untouched (the stores rely on the hardware's range
    check)."""
    tt = L.torch()
    rng = np.random.default_rng(1000 * nk + nq)
    keys = rng.standard_normal((nk, D)).astype(np.float32)
    qs = rng.standard_normal((nq, D)).astype(np.float16)
    codec = tqa.TurboCodec(3, seed=42, projection="gaussian", projection_seed=2)
    packed, sbits, rn = codec.store_qjl(keys)
    idx, g = codec.unpack_codes(packed, 1, nk)
    z = np.unpackbits(np_(sbits), axis=1, bitorder="little")[:, :D].astype(np.float64) * 2 - 1
    ref = O.score_tile(qs.astype(np.float64), np_(idx)[0], np_(g)[0].astype(np.float64), codec.centroids,
                       lambda a: O.rotate_fast(a, codec.signs1, codec.signs2, D), codec.S, z,
                       np_(rn).astype(np.float64), codec.projection_scale)
    scale = np.linalg.norm(qs.astype(np.float64), axis=1).max() * np.linalg.norm(keys.astype(np.float64), axis=1).max()
    for dt, tol in ((tt.float32, 2e-3 * scale / np.sqrt(D) * 4), (tt.float16, 4e-3 * max(np.abs(ref).max(), 1.0))):
        # the logits sit in the middle of a larger buffer filled with a sentinel
        for pad in (64, 1, 3):  # 16-byte aligned, and aligned to the element only (2 or 4, 6 or 12 bytes off)
            buf = tt.full((nq * nk + 2 * pad,), 1024.0, dtype=dt, device="cuda")
            out = buf[pad:pad + nq * nk].view(nq, nk)
            got = codec.score_tile(qs, packed, sbits, rn, nk, out_dtype=dt, out=out)
            assert got.data_ptr() == out.data_ptr()
            a = np_(out).astype(np.float64)
            assert np.abs(a - ref).max() <= tol, (nk, nq, str(dt), pad)
            edge = np_(buf).astype(np.float64)
            assert (edge[:pad] == 1024.0).all() and (edge[pad + nq * nk:] == 1024.0).all()


@pytest.mark.parametrize("bits", [2, 4])
def test_score_tile_other_widths(bits):
    """The estimator tile at the other code widths (their own dequantisation path), fp32 and fp16 logits."""
    tt = L.torch()
    nk, nq = 700, 150
    rng = np.random.default_rng(40 + bits)
    keys = rng.standard_normal((nk, D)).astype(np.float32)
    qs = rng.standard_normal((nq, D)).astype(np.float32)
    codec = tqa.TurboCodec(bits, seed=42, projection="gaussian", projection_seed=5)
    packed, sbits, rn = codec.store_qjl(keys)
    idx, g = codec.unpack_codes(packed, 1, nk)
    z = np.unpackbits(np_(sbits), axis=1, bitorder="little")[:, :D].astype(np.float64) * 2 - 1
    ref = O.score_tile(qs.astype(np.float64), np_(idx)[0], np_(g)[0].astype(np.float64), codec.centroids,
                       lambda a: O.rotate_fast(a, codec.signs1, codec.signs2, D), codec.S, z,
                       np_(rn).astype(np.float64), codec.projection_scale)
    scale = np.linalg.norm(qs.astype(np.float64), axis=1).max() * np.linalg.norm(keys.astype(np.float64), axis=1).max()
    logits = np_(codec.score_tile(qs, packed, sbits, rn, nk)).astype(np.float64)
    assert np.abs(logits - ref).max() <= 2e-3 * scale / np.sqrt(D) * 4
    h = np_(codec.score_tile(qs, packed, sbits, rn, nk, out_dtype=tt.float16)).astype(np.float64)
    assert np.abs(h - ref).max() <= 4e-3 * np.abs(ref).max()


FORMATS = ["turbo2", "turbo3", "turbo4", "q8_0"]


@pytest.mark.parametrize("vfmt", FORMATS)
@pytest.mark.parametrize("kfmt", FORMATS)
def test_decode_attention_every_format_pair(kfmt, vfmt):
    """Every K format with every V format that a layer-adaptive policy can ask for (policy.layer_formats):
    dense and Sparse V, a ragged context, two workgroups' worth of splits."""
    B, Hq, Hkv, N, n_splits = 2, 8, 2, 1100, 4
    rng = np.random.default_rng(FORMATS.index(kfmt) * 4 + FORMATS.index(vfmt))
    k = rng.standard_normal((B * Hkv, N, D)).astype(np.float16)
    v = rng.standard_normal((B * Hkv, N, D)).astype(np.float16)
    q = rng.standard_normal((B, Hq, D)).astype(np.float16)
    kc = tqa.TurboCodec(int(kfmt[-1]), seed=42) if kfmt != "q8_0" else None
    vc = tqa.TurboCodec(int(vfmt[-1]), seed=542) if vfmt != "q8_0" else None
    kp = kc.store(k, kind="k") if kc else tqa.q8_0_store(k)[0]
    vp = vc.store(v, kind="v") if vc else tqa.q8_0_store(v, kind="v")[0]
    for tau in (0.0, 1e-3):
        attn = tqa.DecodeAttention(kc, vc, B, Hq, Hkv, N, n_splits=n_splits, sparse_v_tau=tau)
        out = np_(attn(q, kp, vp))
        ref, skip_o, _ = reference_attention(q, kc, vc, kp, vp, B, Hq, Hkv, N, 1 / np.sqrt(D), n_splits=n_splits, tau=tau,
                                             k_q8=None if kc else kp, v_q8=None if vc else vp)
        assert_close(out, ref)
        if tau:
            assert abs(attn.skip_rate() - skip_o) <= 0.02 * max(skip_o, 1e-3) + 1e-4


@pytest.mark.parametrize("bits,n_splits,Hq", [(3, 12, 64), (4, 24, 64), (2, 12, 40), (3, 36, 48)])
def test_decode_attention_eight_heads_in_workgroups_of_twelve(bits, n_splits, Hq):
    """Eight heads per pass on turbo K and V rows with a split count that is a multiple of 12 and enough groups to
    fill the chip: workgroups of twelve wavefronts (three per SIMD).  Dense, Sparse V, a dense bias; a call with a
    bias list on the same object runs workgroups of eight or four (more partials per group, in the workspace sized at
    construction).  Checked on a sample of the sequences."""
    B, Hkv, N = 32, 8, 1500
    tt = L.torch()
    g = tt.Generator(device="cuda").manual_seed(bits * 100 + n_splits)
    k = tt.randn((B * Hkv, N, D), generator=g, device="cuda").to(tt.float16)
    v = tt.randn((B * Hkv, N, D), generator=g, device="cuda").to(tt.float16)
    # (2-bit rows with queries 1.5 times as long sit at 1.2 times the fp16 bar with every workgroup shape: the rows'
    # few large centroids times a peaked softmax)
    q = ((1.5 if bits > 2 else 1.0) * tt.randn((B, Hq, D), generator=g, device="cuda")).to(tt.float16)
    kc, vc = tqa.TurboCodec(bits, seed=42), tqa.TurboCodec(bits, seed=542)
    kp, vp = kc.store(k, kind="k"), vc.store(v, kind="v")
    bias = tt.zeros((B, Hq, N), dtype=tt.float32, device="cuda")
    bias[:, :, :4] = 2.0
    bias[:, 1::2, N - 1] = -1.5
    per = tqa.packed_bytes(bits, Hkv, N)
    sample = (0, 7, B - 1)

    def check(out, tau, bias_np, skip=None):
        for b in sample:
            bb = None if bias_np is None else bias_np[b:b + 1]
            ref, sk, _ = reference_attention(np_(q[b:b + 1]), kc, vc, kp[b * per:(b + 1) * per], vp[b * per:(b + 1) * per], 1, Hq, Hkv,
                                             N, 1 / np.sqrt(D), n_splits=n_splits, tau=tau, bias=bb)
            assert_close(out[b:b + 1], ref)
        assert np.isfinite(out).all()

    dense = tqa.DecodeAttention(kc, vc, B, Hq, Hkv, N, n_splits=n_splits, poison_output=True)
    check(np_(dense(q, kp, vp)).copy(), 0.0, None)
    bias_np = np_(bias).astype(np.float64)
    check(np_(dense(q, kp, vp, bias=bias)).copy(), 0.0, bias_np)
    check(np_(dense(q, kp, vp, sparse_bias=tqa.sparse_bias_from_dense(bias))).copy(), 0.0, bias_np)
    check(np_(dense(q, kp, vp)).copy(), 0.0, None)                       # and back to the wide workgroups
    sparse = tqa.DecodeAttention(kc, vc, B, Hq, Hkv, N, n_splits=n_splits, sparse_v_tau=1e-3, poison_output=True)
    check(np_(sparse(q, kp, vp)).copy(), 1e-3, None)
    assert 0.0 < sparse.skip_rate() < 1.0
    # the default split count of such a shape is a multiple of 12 when the step is large enough
    assert tqa.turbo.default_splits(128, 32768, eight_heads=True) == 24
    assert tqa.turbo.default_splits(128, 32768, eight_heads=True, turbo_rows=False) == 16
    assert tqa.turbo.default_splits(64, 32768, eight_heads=True) == 32


@pytest.mark.parametrize("kfmt,vfmt", [("turbo3", "turbo3"), ("turbo4", "turbo2"), ("q8_0", "turbo2"), ("q8_0", "q8_0"), ("turbo3", "q8_0"),
                                       ("turbo2", "turbo4")])
def test_decode_attention_eight_heads_per_kv_head(kfmt, vfmt):
    """GQA groups of eight (one pass of two sets of four heads over the same K/V rows) for the table and the int8
    variants, dense and Sparse V with a bias, ragged context, splits that do and do not fill a workgroup."""
    B, Hkv, G, N = 2, 2, 8, 2048 + 100
    Hq = G * Hkv
    rng = np.random.default_rng(FORMATS.index(kfmt) * 7 + FORMATS.index(vfmt))
    k = rng.standard_normal((B * Hkv, N, D)).astype(np.float16)
    v = rng.standard_normal((B * Hkv, N, D)).astype(np.float16)
    q = rng.standard_normal((B, Hq, D)).astype(np.float16)
    bias = (0.7 * rng.standard_normal((B, Hq, N))).astype(np.float32)
    bias_d = L.torch().from_numpy(bias).cuda()
    kc = tqa.TurboCodec(int(kfmt[-1]), seed=42) if kfmt != "q8_0" else None
    vc = tqa.TurboCodec(int(vfmt[-1]), seed=542) if vfmt != "q8_0" else None
    kp = kc.store(k, kind="k") if kc else tqa.q8_0_store(k)[0]
    vp = vc.store(v, kind="v") if vc else tqa.q8_0_store(v, kind="v")[0]
    for n_splits, tau in ((8, 0.0), (24, 1e-3), (3, 1e-3)):
        attn = tqa.DecodeAttention(kc, vc, B, Hq, Hkv, N, n_splits=n_splits, sparse_v_tau=tau)
        out = np_(attn(q, kp, vp, bias=bias_d))
        ref, skip_o, _ = reference_attention(q, kc, vc, kp, vp, B, Hq, Hkv, N, 1 / np.sqrt(D), n_splits=n_splits, tau=tau,
                                             bias=bias, k_q8=None if kc else kp, v_q8=None if vc else vp)
        assert_close(out, ref)
        if tau:
            assert abs(attn.skip_rate() - skip_o) <= 0.02 * max(skip_o, 1e-3) + 1e-4
            assert int(attn.skip.cpu()[1]) == B * Hq * N
