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
from turboquant_plus_amd.turbo import OVERRUN_NEGATIVE, OVERRUN_NO_ROOM, overrun_bits
from test_gpu_turbo import check_codes, np_

pytestmark = pytest.mark.gpu
D = 128


def blocks_of(buf, bits, n_seqs, capacity):
    return np_(buf).reshape(n_seqs, -1, O.block_bytes(bits))


@pytest.mark.parametrize("bits", [2, 3, 4])
@pytest.mark.parametrize("kind", ["k", "v"])
def test_append_in_chunks_equals_store(bits, kind):
    """float64 rows: tq_store serves them with the butterfly arithmetic that tq_append uses, so the bytes are equal
    (fp16 and fp32 rows are stored through the matrix cores, whose codes agree with the append's outside the boundary
    band: test_append_codes_match_oracle, test_prefill_into_a_cache_laid_out_for_more_tokens)."""
    tt = L.torch()
    codec = tqa.TurboCodec(bits, seed=7)
    n_seqs, capacity = 3, 512
    x = np.random.default_rng(bits).standard_normal((n_seqs, 300, D)).astype(np.float32).astype(np.float64)
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


@pytest.mark.parametrize("bits", [2, 3, 4])
@pytest.mark.parametrize("kind", ["k", "v"])
@pytest.mark.parametrize("back_to,n_new", [(150, 1), (130, 17), (64, 3), (13, 1), (127, 2)])
def test_append_after_a_rewind_truncates(bits, kind, back_to, n_new):
    """Appending at a position below the tokens already written (a rolled-back speculative step) leaves
    the touched blocks as tq_store writes them for the shortened sequence: the stale tokens behind the
    new ones are gone from those blocks."""
    tt = L.torch()
    codec = tqa.TurboCodec(bits, seed=9)
    n_seqs, capacity = 2, 384
    rng = np.random.default_rng(bits * 100 + back_to)
    x = rng.standard_normal((n_seqs, 230, D)).astype(np.float32).astype(np.float64)   # float64 rows: see above
    y = rng.standard_normal((n_seqs, n_new, D)).astype(np.float32).astype(np.float64)
    cache = tt.zeros(tqa.packed_bytes(bits, n_seqs, capacity), dtype=tt.uint8, device="cuda")
    codec.append(x, cache, 0, capacity, kind=kind)
    codec.append(y, cache, back_to, capacity, kind=kind)
    now = np.concatenate([x[:, :back_to], y], axis=1)
    want = np_(codec.store(now, kind=kind)).reshape(n_seqs, -1, O.block_bytes(bits))
    got = blocks_of(cache, bits, n_seqs, capacity)
    first, last = back_to // 128, (back_to + n_new - 1) // 128
    for b in range(first, last + 1):      # the blocks the second append touched
        assert np.array_equal(got[:, b], want[:, b]), f"block {b}"
    for b in range(first):                # blocks before it are untouched
        assert np.array_equal(got[:, b], want[:, b]), f"block {b}"


@pytest.mark.parametrize("kbits,vbits", [(3, 3), (4, 4), (4, 2), (2, 4)])
def test_append_kv_equals_two_appends(kbits, vbits):
    """K and V of a step in one launch (tq_append_kv) write the bytes of two tq_append calls;
    the (2, 4) pair has no fused kernel and takes the two-launch route inside the library."""
    tt = L.torch()
    kc, vc = tqa.TurboCodec(kbits, seed=7), tqa.TurboCodec(vbits, seed=507)
    n_seqs, capacity = 5, 384
    rng = np.random.default_rng(kbits * 10 + vbits)
    k = rng.standard_normal((n_seqs, 200, D)).astype(np.float16)
    v = rng.standard_normal((n_seqs, 200, D)).astype(np.float16)
    ck = tt.zeros(tqa.packed_bytes(kbits, n_seqs, capacity), dtype=tt.uint8, device="cuda")
    cv = tt.zeros(tqa.packed_bytes(vbits, n_seqs, capacity), dtype=tt.uint8, device="cuda")
    rk, rv = tt.zeros_like(ck), tt.zeros_like(cv)
    pos = 0
    for n_new in [1, 1, 126, 1, 70, 1]:
        kc.append_kv(vc, k[:, pos:pos + n_new], v[:, pos:pos + n_new], ck, cv, pos, capacity)
        kc.append(k[:, pos:pos + n_new], rk, pos, capacity, kind="k")
        vc.append(v[:, pos:pos + n_new], rv, pos, capacity, kind="v")
        pos += n_new
        assert tt.equal(ck, rk) and tt.equal(cv, rv), f"after {pos} tokens"
    with pytest.raises(ValueError):
        kc.append_kv(vc, k[:, :2], v[:, :3], ck, cv, 0, capacity)


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


# ---- temporal decay: re-quantise packed rows to a narrower codebook ---------------------------

def _check_requant(src, dst, packed_src, n_seqs, tokens, kind):
    idx_s, g_s = src.unpack_codes(packed_src, n_seqs, tokens, kind=kind)
    out = src.requantize_to(dst, packed_src, n_seqs, tokens, kind=kind)
    assert out.numel() == tqa.packed_bytes(dst.bits, n_seqs, tokens)
    idx_d, g_d = dst.unpack_codes(out, n_seqs, tokens, kind=kind)
    idx_s, g_s = np_(idx_s).reshape(-1, D), np_(g_s).reshape(-1).astype(np.float64)
    idx_d, g_d = np_(idx_d).reshape(-1, D), np_(g_d).reshape(-1)
    want_idx, want_g = O.requantize(idx_s, g_s, src.centroids, dst.centroids)
    # decision values of the oracle, for the boundary-band accounting of mismatching codes
    vals = src.centroids[idx_s] * g_s[:, None]
    nrm = np.linalg.norm(vals, axis=1, keepdims=True)
    y = np.where(nrm > 1e-10, vals / np.where(nrm > 1e-10, nrm, 1.0), vals)
    live = g_s != 0                                     # rows of all-zero vectors decode to 0 whatever their codes
    n_bad, n_inadm = O.boundary_band_mismatches(y[live], idx_d[live], dst.centroids, rel=1e-6)
    assert n_inadm == 0 and n_bad <= max(2, 2e-5 * idx_d.size)
    same = np.all(idx_d == want_idx, axis=1)
    a = g_d.astype(np.float16)[same].view(np.uint16).astype(np.int32)
    b = want_g.astype(np.float16)[same].view(np.uint16).astype(np.int32)
    assert np.abs(a - b).max(initial=0) <= 1 and (np.abs(a - b) == 1).sum() <= max(2, 2e-3 * a.size)
    assert np.all(g_d[~live] == 0)
    return out


def test_decode_step_replayed_from_a_hip_graph():
    """append_kv + decode attention (dense and Sparse V) captured once in a HIP graph and replayed with new
    inputs: every replay equals the eager result bit for bit, with eager work between the replays."""
    tt = L.torch()
    B, Hq, Hkv, cap, pos = 2, 8, 2, 512, 300
    kc, vc = tqa.TurboCodec(3, seed=42), tqa.TurboCodec(3, seed=542)
    rng = np.random.default_rng(5)
    k0 = rng.standard_normal((B * Hkv, pos, D)).astype(np.float16)
    v0 = rng.standard_normal((B * Hkv, pos, D)).astype(np.float16)
    ck = tt.zeros(tqa.packed_bytes(3, B * Hkv, cap), dtype=tt.uint8, device="cuda")
    cv = tt.zeros_like(ck)
    kc.append_kv(vc, k0, v0, ck, cv, 0, cap)
    base_k, base_v = ck.clone(), cv.clone()
    q_s = tt.zeros((B, Hq, D), dtype=tt.float16, device="cuda")
    kn_s = tt.zeros((B * Hkv, 1, D), dtype=tt.float16, device="cuda")
    vn_s = tt.zeros_like(kn_s)
    for tau in (0.0, 1e-3):
        attn = tqa.DecodeAttention(kc, vc, B, Hq, Hkv, pos + 1, n_splits=4, capacity=cap, sparse_v_tau=tau)

        def step():
            kc.append_kv(vc, kn_s, vn_s, ck, cv, pos, cap)
            return attn(q_s, ck, cv)

        side = tt.cuda.Stream()
        side.wait_stream(tt.cuda.current_stream())
        with tt.cuda.stream(side):
            step()                                   # warm-up outside the capture
        tt.cuda.current_stream().wait_stream(side)
        graph = tt.cuda.CUDAGraph()
        with tt.cuda.graph(graph):
            out_g = step()
        for trial in range(4):
            q = tt.from_numpy(rng.standard_normal((B, Hq, D)).astype(np.float16)).cuda()
            kn = tt.from_numpy(rng.standard_normal((B * Hkv, 1, D)).astype(np.float16)).cuda()
            vn = tt.from_numpy(rng.standard_normal((B * Hkv, 1, D)).astype(np.float16)).cuda()
            ek, ev = base_k.clone(), base_v.clone()      # eager reference on private buffers
            kc.append_kv(vc, kn, vn, ek, ev, pos, cap)
            eager = tqa.DecodeAttention(kc, vc, B, Hq, Hkv, pos + 1, n_splits=4, capacity=cap, sparse_v_tau=tau)
            want = eager(q, ek, ev).clone()
            want_skip = eager.skip_rate() if tau else 0.0
            tt.cuda.synchronize()
            q_s.copy_(q)
            kn_s.copy_(kn)
            vn_s.copy_(vn)
            graph.replay()
            tt.cuda.synchronize()
            assert tt.equal(out_g, want), f"tau {tau}, replay {trial}"
            assert tt.equal(ck, ek) and tt.equal(cv, ev)
            if tau:
                assert attn.skip_rate() == want_skip


def test_requantize_3_to_2_prototype_presets(golden):
    """The prototype's literal centroid presets, its rows, device format in between."""
    c3, c2 = golden["decay_c3"], golden["decay_c2"]
    src, dst = tqa.TurboCodec(3, seed=9, centroids=c3), tqa.TurboCodec(2, seed=9, centroids=c2)
    idx3 = np.zeros((128, D), dtype=np.uint8)
    idx3[:48] = golden["decay_idx3"]
    g3 = np.zeros(128, dtype=np.float16)
    g3[:48] = (golden["decay_norm3"] / np.sqrt(np.sum(c3[golden["decay_idx3"]] ** 2, axis=1))).astype(np.float16)
    for kind in ("k", "v"):
        packed = L.torch().from_numpy(O.layout_pack(idx3, g3, 3, kind)).cuda()
        out = _check_requant(src, dst, packed, 1, 128, kind)
        i2, g2 = O.layout_unpack(np_(out), 2, kind)
        assert np.array_equal(i2[:48], golden["decay_idx2"])          # fp16 norms do not move these decisions


@pytest.mark.parametrize("pair", [(3, 2), (4, 3), (4, 2)])
@pytest.mark.parametrize("kind", ["k", "v"])
def test_requantize_stored_cache(pair, kind):
    sb, db = pair
    src, dst = tqa.TurboCodec(sb, seed=42), tqa.TurboCodec(db, seed=42)
    x = np.random.default_rng(sb * 10 + db).standard_normal((3, 200, D)).astype(np.float16)
    x[2, 7] = 0
    packed = src.store(x, kind=kind)
    out = _check_requant(src, dst, packed, 3, 200, kind)
    # decayed rows still reconstruct the input: error between the two widths' own errors
    rec_s = np_(src.load(packed, 3, 200, kind=kind, domain="original"))
    rec_d = np_(dst.load(out, 3, 200, kind=kind, domain="original"))
    direct = np_(dst.load(dst.store(x, kind=kind), 3, 200, kind=kind, domain="original"))
    xf = x.astype(np.float64)
    err = lambda r: float(np.mean(np.sum((r - xf) ** 2, -1)) / np.mean(np.sum(xf ** 2, -1)))
    assert err(rec_s) < err(rec_d) < 1.6 * err(direct)


@pytest.mark.parametrize("pair", [(3, 2), (4, 3), (4, 2)])
@pytest.mark.parametrize("kind", ["k", "v"])
def test_requantize_rows_whose_code_map_is_their_own(pair, kind):
    """Rows go through a code -> code table that holds for rows whose sum of squared centroids lies in an interval
    around 1; other rows build their own table (K: the row's lane; V: the token's lane, and every lane of the tile
    re-maps its two codes of that token).  Rows drawn from a random subset of the levels (all outer levels, all
    inner levels, one level only, ...) have sums between 0.2 and 5 and maps that differ from the common one - an outer
    level that falls into an inner cell once the row is renormalised - and rows with norm zero take the same path.
    Five blocks: the launch's workgroups serve eight at a time, so a ragged last set is covered too."""
    sb, db = pair
    src, dst = tqa.TurboCodec(sb, seed=42), tqa.TurboCodec(db, seed=42)
    rng = np.random.default_rng(100 * sb + db)
    tokens = 5 * 128
    idx = np.zeros((tokens, D), dtype=np.uint8)
    sums = np.zeros(tokens)
    for r in range(tokens):
        levels = np.flatnonzero(rng.random(1 << sb) < 0.4)
        if levels.size == 0:
            levels = np.array([rng.integers(1 << sb)])
        idx[r] = rng.choice(levels, size=D)
        sums[r] = np.sum(src.centroids[idx[r]] ** 2)
    assert sums.min() < 0.5 and sums.max() > 3.0
    g = rng.uniform(0.01, 30.0, tokens).astype(np.float16)
    g[rng.integers(0, tokens, 7)] = 0
    packed = L.torch().from_numpy(O.layout_pack(idx, g, sb, kind)).cuda()
    out = _check_requant(src, dst, packed, 1, tokens, kind)
    # the maps do differ: many rows do not get the codes a unit-sum row would
    common = np.searchsorted(O.midpoints(dst.centroids), src.centroids, side="right")
    i2, _ = O.layout_unpack(np_(out), db, kind)
    live = g != 0
    assert np.mean(np.any(i2[:tokens][live] != common[idx][live], axis=1)) > 0.2


def test_requantize_rejects_widening():
    a, b = tqa.TurboCodec(2, seed=1), tqa.TurboCodec(3, seed=1)
    buf = L.torch().zeros(tqa.packed_bytes(2, 1, 128), dtype=L.torch().uint8, device="cuda")
    with pytest.raises(NotImplementedError):
        a.requantize_to(b, buf, 1, 128)


# ---- interchange with the fork's per-128 block layout ------------------------------------------

@pytest.mark.parametrize("bits", [2, 3, 4])
@pytest.mark.parametrize("kind", ["k", "v"])
def test_fork_blocks_export_import(bits, kind):
    codec = tqa.TurboCodec(bits, seed=42, centroids=tqa.PRODUCTION_CENTROIDS[bits])
    n_seqs, tokens = 3, 200
    x = np.random.default_rng(bits).standard_normal((n_seqs, tokens, D)).astype(np.float16)
    x[0, 9] = 0
    packed = codec.store(x, kind=kind)
    idx, g = codec.unpack_codes(packed, n_seqs, tokens, kind=kind)
    idx, g = np_(idx).reshape(-1, D), np_(g).reshape(-1)
    check_codes(codec, x.reshape(-1, D), idx, g)                      # the fork's centroid tables quantise like any other
    blocks = codec.export_fork_blocks(packed, n_seqs, tokens, kind=kind)
    assert tuple(blocks.shape) == (n_seqs, tokens, O.fork_block_bytes(bits))
    want = O.fork_blocks_pack(idx, g.astype(np.float16), bits).reshape(n_seqs, tokens, -1)
    assert np.array_equal(np_(blocks), want)
    back = codec.import_fork_blocks(blocks, kind=kind)
    assert np.array_equal(np_(back), np_(packed))                     # including the padding rows of the last block
    # blocks written elsewhere (here: by the oracle from random codes) come in as the same codes
    rng = np.random.default_rng(1)
    ridx = rng.integers(0, 1 << bits, size=(2 * 128, D)).astype(np.uint8)
    rg = np.abs(rng.standard_normal(2 * 128)).astype(np.float16)
    ext = O.fork_blocks_pack(ridx, rg, bits).reshape(2, 128, -1)
    if bits == 4:
        assert ext.shape[2] == 68 and (np_(blocks)[:, :, 2:4] == 0).all()   # 4.25 bits per value; rnorm exported as 0
        ext[:, :, 2:4] = 0x5A                                                # and ignored on the way in
    i2, g2 = codec.unpack_codes(codec.import_fork_blocks(ext, kind=kind), 2, 128, kind=kind)
    assert np.array_equal(np_(i2).reshape(-1, D), ridx) and np.array_equal(np_(g2).reshape(-1).astype(np.float16), rg)


@pytest.mark.parametrize("bits", [2, 3, 4])
@pytest.mark.parametrize("kind", ["k", "v"])
def test_fork_blocks_and_requantize_at_config_2_size(bits, kind):
    """262 144 vectors (8 heads x 32768 tokens, the store configuration): export followed by import gives the packed
    buffer back byte for byte; sampled rows of the export equal the oracle's packing of the unpacked codes; and a
    requantised buffer decodes, on sampled rows, to the codes the oracle's requantisation of those rows gives."""
    tt = L.torch()
    heads, tokens = 8, 32768
    codec = tqa.TurboCodec(bits, seed=42)
    g = tt.Generator(device="cuda").manual_seed(50 + bits)
    x = tt.randn((heads, tokens, D), generator=g, device="cuda").to(tt.float16)
    packed = codec.store(x, kind=kind)
    blocks = codec.export_fork_blocks(packed, heads, tokens, kind=kind)
    assert tt.equal(codec.import_fork_blocks(blocks, kind=kind), packed)
    idx, gn = codec.unpack_codes(packed, heads, tokens, kind=kind)
    rows = np.random.default_rng(bits).integers(0, heads * tokens, size=256)
    idx_s = np_(idx).reshape(-1, D)[rows]
    g_s = np_(gn).reshape(-1)[rows].astype(np.float16)
    assert np.array_equal(np_(blocks).reshape(heads * tokens, -1)[rows], O.fork_blocks_pack(idx_s, g_s, bits))
    if bits > 2:
        dst = tqa.TurboCodec(bits - 1, seed=42)
        narrow = codec.requantize_to(dst, packed, heads, tokens, kind=kind)
        i2, g2 = dst.unpack_codes(narrow, heads, tokens, kind=kind)
        want_i, want_g = O.requantize(idx_s, g_s.astype(np.float32), codec.centroids, dst.centroids)
        got_i = np_(i2).reshape(-1, D)[rows]
        assert (got_i != want_i).mean() < 1e-4                       # fp32 on the device, float64 in the oracle: boundary cases
        assert np.allclose(np_(g2).reshape(-1)[rows], want_g, rtol=2e-3)


@pytest.mark.parametrize("bits", [2, 3, 4])
@pytest.mark.parametrize("kind", ["k", "v"])
def test_fork_blocks_at_the_least_alignment(bits, kind):
    """Fork rows that start 2 bytes (4 for 68-byte rows) past a 16-byte boundary and sequences of 77 tokens, whose rows
    start at every even residue: the K kernels move whole 16-byte pieces where the address allows and 2-byte pieces
    around them, and must write nothing outside the rows."""
    tt = L.torch()
    codec = tqa.TurboCodec(bits, seed=42)
    n_seqs, tokens, fb = 3, 77, O.fork_block_bytes(bits)
    x = np.random.default_rng(40 + bits).standard_normal((n_seqs, tokens, D)).astype(np.float16)
    packed = codec.store(x, kind=kind)
    idx, g = codec.unpack_codes(packed, n_seqs, tokens, kind=kind)
    want = O.fork_blocks_pack(np_(idx).reshape(-1, D), np_(g).reshape(-1).astype(np.float16), bits).reshape(-1)
    off = 4 if bits == 4 else 2
    raw = tt.full((off + want.size + 64,), 0xA5, dtype=tt.uint8, device="cuda")
    lib = L.lib()
    knd = L.KIND_K if kind == "k" else L.KIND_V
    rc = lib.tq_export_fork_blocks(codec.handle.h, L.ptr(packed), n_seqs, tokens, knd, L.ptr(raw[off:]), L.stream_ptr())
    assert rc == 0
    got = np_(raw)
    assert np.array_equal(got[off:off + want.size], want)
    assert (got[:off] == 0xA5).all() and (got[off + want.size:] == 0xA5).all()
    back = tt.full_like(packed, 0x3C)
    rc = lib.tq_import_fork_blocks(codec.handle.h, L.ptr(raw[off:]), n_seqs, tokens, knd, L.ptr(back), L.stream_ptr())
    assert rc == 0
    assert tt.equal(back, packed)


@pytest.mark.parametrize("bits", [2, 3])
@pytest.mark.parametrize("kind", ["k", "v"])
@pytest.mark.parametrize("block_values", [32, 64])
def test_fork_blocks_of_32_and_64_values(bits, kind, block_values):
    """Caches of the fork's earlier builds (storage blocks of 32 values, 64 measured too;
    docs/papers/block-size-experiment.md:27-39): the export equals the oracle's packing block by block with the group's
    norm in every block, the import gives the packed buffer back byte for byte (ragged last block included) and reads
    the first block's norm; rows at the least alignment write nothing outside themselves."""
    tt = L.torch()
    codec = tqa.TurboCodec(bits, seed=42, centroids=tqa.PRODUCTION_CENTROIDS[bits])
    n_seqs, tokens = 3, 205
    x = np.random.default_rng(7 * bits + block_values).standard_normal((n_seqs, tokens, D)).astype(np.float16)
    x[1, 17] = 0
    packed = codec.store(x, kind=kind)
    idx, g = codec.unpack_codes(packed, n_seqs, tokens, kind=kind)
    idx, g = np_(idx).reshape(-1, D), np_(g).reshape(-1).astype(np.float16)
    rb = O.fork_row_bytes(bits, block_values)
    assert L.lib().tq_fork_row_bytes(bits, block_values) == rb
    blocks = codec.export_fork_blocks(packed, n_seqs, tokens, kind=kind, block_values=block_values)
    assert tuple(blocks.shape) == (n_seqs, tokens, rb)
    want = O.fork_blocks_pack(idx, g, bits, block_values)
    assert np.array_equal(np_(blocks).reshape(-1, rb), want)
    assert tt.equal(codec.import_fork_blocks(blocks, kind=kind, block_values=block_values), packed)
    # blocks written elsewhere: random codes; the later blocks of a vector carry another norm, which nobody reads
    rng = np.random.default_rng(block_values)
    ridx = rng.integers(0, 1 << bits, size=(2 * 128, D)).astype(np.uint8)
    rg = np.abs(rng.standard_normal(2 * 128)).astype(np.float16)
    ext = O.fork_blocks_pack(ridx, rg, bits, block_values).reshape(2 * 128, 128 // block_values, -1)
    ext[:, 1:, 0:2] = 0x3C
    i2, g2 = codec.unpack_codes(codec.import_fork_blocks(ext.reshape(2, 128, rb), kind=kind, block_values=block_values),
                                2, 128, kind=kind)
    assert np.array_equal(np_(i2).reshape(-1, D), ridx) and np.array_equal(np_(g2).reshape(-1).astype(np.float16), rg)
    # 2 bytes past a 16-byte boundary, 77 tokens per sequence
    tokens = 77
    packed = codec.store(x[:, :tokens], kind=kind)
    idx, g = codec.unpack_codes(packed, n_seqs, tokens, kind=kind)
    want = O.fork_blocks_pack(np_(idx).reshape(-1, D), np_(g).reshape(-1).astype(np.float16), bits, block_values).reshape(-1)
    raw = tt.full((2 + want.size + 64,), 0xA5, dtype=tt.uint8, device="cuda")
    lib = L.lib()
    knd = L.KIND_K if kind == "k" else L.KIND_V
    rc = lib.tq_export_fork_blocks_sized(codec.handle.h, L.ptr(packed), n_seqs, tokens, knd, block_values, L.ptr(raw[2:]),
                                         L.stream_ptr())
    assert rc == 0
    got = np_(raw)
    assert np.array_equal(got[2:2 + want.size], want)
    assert (got[:2] == 0xA5).all() and (got[2 + want.size:] == 0xA5).all()
    back = tt.full_like(packed, 0x3C)
    rc = lib.tq_import_fork_blocks_sized(codec.handle.h, L.ptr(raw[2:]), n_seqs, tokens, knd, block_values, L.ptr(back),
                                         L.stream_ptr())
    assert rc == 0
    assert tt.equal(back, packed)


def test_fork_blocks_refuse_a_block_size_the_fork_lacks():
    tt = L.torch()
    c4, c3 = tqa.TurboCodec(4, seed=42), tqa.TurboCodec(3, seed=42)
    p4 = c4.store(np.ones((1, 128, D), dtype=np.float16))
    with pytest.raises(ValueError, match="no 4-bit layout with 32 values"):
        c4.export_fork_blocks(p4, 1, 128, block_values=32)
    with pytest.raises(ValueError, match="no 3-bit layout with 16 values"):
        c3.import_fork_blocks(np.zeros((1, 128, 50), dtype=np.uint8), block_values=16)
    out = tt.zeros(128 * 68, dtype=tt.uint8, device="cuda")
    rc = L.lib().tq_export_fork_blocks_sized(c4.handle.h, L.ptr(p4), 1, 128, L.KIND_K, 64, L.ptr(out), L.stream_ptr())
    assert rc == L.ERR_UNSUPPORTED and "not a layout of the fork" in L.last_error()
    assert not np_(out).any()


def test_fork_blocks_rejects_wrong_width():
    codec = tqa.TurboCodec(3, seed=42)
    with pytest.raises(ValueError):
        codec.import_fork_blocks(np.zeros((1, 128, 66), dtype=np.uint8))


def test_fork_blocks_reject_an_odd_address():
    """A fork block starts with its fp16 norm and every block size is even: the kernels read and write rows as
    16-bit pieces, so a blocks buffer at an odd address is refused (TQ_ERR_ALIGN) before anything is launched."""
    tt = L.torch()
    codec = tqa.TurboCodec(3, seed=42)
    packed = codec.store(np.random.default_rng(3).standard_normal((1, 128, D)).astype(np.float16))
    raw = tt.zeros(128 * 50 + 2, dtype=tt.uint8, device="cuda")
    lib = L.lib()
    rc = lib.tq_export_fork_blocks(codec.handle.h, L.ptr(packed), 1, 128, L.KIND_K, L.ptr(raw[1:]), L.stream_ptr())
    assert rc == L.ERR_ALIGN
    rc = lib.tq_import_fork_blocks(codec.handle.h, L.ptr(raw[1:]), 1, 128, L.KIND_K, L.ptr(packed), L.stream_ptr())
    assert rc == L.ERR_ALIGN
    assert (np_(raw) == 0).all()
    # 4-bit blocks (68 bytes: norm, rnorm, sixteen 4-byte code words) move as 4-byte words
    codec4 = tqa.TurboCodec(4, seed=42)
    packed4 = codec4.store(np.random.default_rng(3).standard_normal((1, 128, D)).astype(np.float16))
    raw4 = tt.zeros(128 * 68 + 4, dtype=tt.uint8, device="cuda")
    rc = lib.tq_export_fork_blocks(codec4.handle.h, L.ptr(packed4), 1, 128, L.KIND_K, L.ptr(raw4[2:]), L.stream_ptr())
    assert rc == L.ERR_ALIGN
    rc = lib.tq_import_fork_blocks(codec4.handle.h, L.ptr(raw4[2:]), 1, 128, L.KIND_K, L.ptr(packed4), L.stream_ptr())
    assert rc == L.ERR_ALIGN
    assert (np_(raw4) == 0).all()


# ---- q8_0-style buffers (boundary layers of a layer-adaptive policy) ---------------------------------------

@pytest.mark.parametrize("kind", ["k", "v"])
@pytest.mark.parametrize("dtype", [np.float16, np.float32])
def test_q8_0_append_in_chunks_equals_store(kind, dtype):
    tt = L.torch()
    n_seqs, capacity = 3, 512
    x = np.random.default_rng(11).standard_normal((n_seqs, 300, D)).astype(dtype)
    x[1, 5] = 0
    cache = tt.zeros(128 * 136 * n_seqs * 4, dtype=tt.uint8, device="cuda")
    pos = 0
    for n_new in [1, 1, 62, 64, 5, 130, 37]:
        tqa.q8_0_append(x[:, pos:pos + n_new], cache, pos, capacity, kind=kind)
        pos += n_new
        want = np_(tqa.q8_0_store(x[:, :pos], kind=kind)[0]).reshape(n_seqs, -1, 128 * 136)
        got = np_(cache).reshape(n_seqs, -1, 128 * 136)
        nb = want.shape[1]
        assert np.array_equal(got[:, :nb], want), f"after {pos} tokens"
        assert not got[:, nb:].any()
    # a rewind truncates: the touched block holds the tokens before pos, the new ones, then zeros
    tqa.q8_0_append(x[:, 100:103], cache, 200, capacity, kind=kind)
    y = np.concatenate([x[:, :200], x[:, 100:103]], axis=1)
    want = np_(tqa.q8_0_store(y, kind=kind)[0]).reshape(n_seqs, -1, 128 * 136)
    got = np_(cache).reshape(n_seqs, -1, 128 * 136)
    assert np.array_equal(got[:, :2], want)
    with pytest.raises(ValueError):
        tqa.q8_0_append(x[:, :10], cache, 510, capacity, kind=kind)


@pytest.mark.parametrize("fmt", [("q8_0", "q8_0"), ("q8_0", "turbo2"), ("turbo3", "q8_0"), ("turbo3", "turbo3")])
def test_layer_decode_loop_over_a_growing_cache(fmt):
    """A layer of a layer-adaptive policy in a serving loop: prefill by one append, then single-token appends with
    attention after each, against attention over a cache stored in one go."""
    from test_gpu_attention import assert_close, reference_attention
    B, Hq, Hkv, capacity = 2, 8, 2, 400
    layer = tqa.LayerKV(tqa.LayerFormat(*fmt), seed=3)
    rng = np.random.default_rng(12)
    # fp32 input: the append and the store of fp32 rows share one arithmetic (fp16 rows are stored through the
    # matrix-core rotation, which may round a value at a code boundary the other way)
    k = rng.standard_normal((B * Hkv, 260, D)).astype(np.float32)
    v = rng.standard_normal((B * Hkv, 260, D)).astype(np.float32)
    kc, vc = layer.new_cache(B * Hkv, capacity)
    attn = layer.attention(B, Hq, Hkv, 1, n_splits=2, capacity=capacity)
    layer.append(k[:, :250], v[:, :250], kc, vc, 0, capacity)
    pos = 250
    for step in range(10):
        layer.append(k[:, pos:pos + 1], v[:, pos:pos + 1], kc, vc, pos, capacity)
        pos += 1
        q = rng.standard_normal((B, Hq, D)).astype(np.float16)
        attn.set_tokens(pos)
        out = np_(attn(q, kc, vc)).copy()
        kp, vp = layer.store(k[:, :pos], v[:, :pos])
        once = np_(layer.attention(B, Hq, Hkv, pos, n_splits=2)(q, kp, vp))
        assert np.array_equal(out, once), f"step {step}"
    ref, _, _ = reference_attention(q, layer.k_codec, layer.v_codec, kp, vp, B, Hq, Hkv, pos, 1 / np.sqrt(D),
                                    k_q8=kp if layer.k_codec is None else None, v_q8=vp if layer.v_codec is None else None)
    assert_close(out, ref)


def test_store_into_a_capacity_buffer_is_rejected_for_several_sequences():
    """tq_store lays sequences out ceil(tokens / 128) blocks apart; a buffer sized for a larger capacity has
    another stride, so the host wrapper refuses it instead of mislaying every sequence after the first."""
    tt = L.torch()
    kc, vc = tqa.TurboCodec(3, seed=42), tqa.TurboCodec(3, seed=542)
    x = np.random.default_rng(0).standard_normal((2, 128, D)).astype(np.float16)
    cache = tt.zeros(tqa.packed_bytes(3, 2, 512), dtype=tt.uint8, device="cuda")
    with pytest.raises(ValueError, match="append"):
        kc.store(x, kind="k", out=cache)
    with pytest.raises(ValueError, match="append_kv"):
        kc.store_kv(vc, x, x, out_k=cache, out_v=cache.clone())
    one = kc.store(x[:1], kind="k", out=cache)           # a single sequence has no stride: allowed
    assert one is cache


@pytest.mark.parametrize("kb,vb", [(3, 3), (4, 4), (3, 2)])
@pytest.mark.parametrize("tokens", [64, 200, 256, 300, 700])
def test_prefill_into_a_cache_laid_out_for_more_tokens(kb, vb, tokens):
    """tq_store_kv_cache: fp16 prompts go through the matrix-core store straight into buffers laid out for `capacity`
    tokens per sequence.  Every sequence's first blocks hold the bytes tq_store_kv writes for it, the other blocks stay
    untouched, and the cache then grows by appends as one that was filled by appends: the prefix is kept bit for bit and
    the appended token gets the same codes."""
    tt = L.torch()
    n_seqs, capacity = 3, 512 if tokens < 500 else 1024
    kc, vc = tqa.TurboCodec(kb, seed=42), tqa.TurboCodec(vb, seed=542)
    rng = np.random.default_rng(100 * kb + tokens)
    k = rng.standard_normal((n_seqs, tokens + 1, D)).astype(np.float16)
    v = rng.standard_normal((n_seqs, tokens + 1, D)).astype(np.float16)
    ck = tt.full((tqa.packed_bytes(kb, n_seqs, capacity),), 0xA5, dtype=tt.uint8, device="cuda")
    cv = tt.full((tqa.packed_bytes(vb, n_seqs, capacity),), 0xA5, dtype=tt.uint8, device="cuda")
    kc.store_kv(vc, k[:, :tokens], v[:, :tokens], out_k=ck, out_v=cv, capacity=capacity)
    pk, pv = kc.store_kv(vc, k[:, :tokens], v[:, :tokens])
    nb = -(-tokens // 128)
    for bits, cache, plain in ((kb, ck, pk), (vb, cv, pv)):
        got = np_(cache).reshape(n_seqs, capacity // 128, -1)
        assert np.array_equal(got[:, :nb], np_(plain).reshape(n_seqs, nb, -1))
        assert (got[:, nb:] == 0xA5).all(), "touched a block past the prompt"
    # grow both this cache and one filled by appends (zeroed, as new_cache() hands them out) by one token
    ak = tt.zeros_like(ck)
    av = tt.zeros_like(cv)
    kc.append_kv(vc, k[:, :tokens], v[:, :tokens], ak, av, 0, capacity)
    for a, b in ((ck, cv), (ak, av)):
        kc.append_kv(vc, k[:, tokens:], v[:, tokens:], a, b, tokens, capacity)
    for codec, kind, mine, theirs, plain in ((kc, "k", ck, ak, pk), (vc, "v", cv, av, pv)):
        idx_m, g_m = (np_(t) for t in codec.unpack_codes(mine, n_seqs, capacity, kind=kind))
        idx_t, g_t = (np_(t) for t in codec.unpack_codes(theirs, n_seqs, capacity, kind=kind))
        idx_p, g_p = (np_(t) for t in codec.unpack_codes(plain, n_seqs, tokens, kind=kind))
        assert np.array_equal(idx_m[:, :tokens], idx_p) and np.array_equal(g_m[:, :tokens], g_p), "the append moved the prefix"
        assert np.array_equal(idx_m[:, tokens], idx_t[:, tokens]) and np.array_equal(g_m[:, tokens], g_t[:, tokens])
        # matrix-core store against butterfly append of the same fp16 rows: the same codes but for values at a boundary
        assert (idx_m[:, :tokens] != idx_t[:, :tokens]).mean() < 1e-4


def test_prefill_falls_back_to_the_append_for_fp64_rows_and_checks_its_arguments():
    """Rows the matrix-core store does not take (float64) reach a cache through the append from position 0."""
    tt = L.torch()
    n_seqs, tokens, capacity = 2, 150, 384
    kc, vc = tqa.TurboCodec(3, seed=42), tqa.TurboCodec(3, seed=542)
    rng = np.random.default_rng(8)
    k = rng.standard_normal((n_seqs, tokens, D))
    v = rng.standard_normal((n_seqs, tokens, D))
    ck, cv = (tt.zeros(tqa.packed_bytes(3, n_seqs, capacity), dtype=tt.uint8, device="cuda") for _ in range(2))
    ak, av = tt.zeros_like(ck), tt.zeros_like(cv)
    kc.store_kv(vc, k, v, out_k=ck, out_v=cv, capacity=capacity)
    kc.append_kv(vc, k, v, ak, av, 0, capacity)
    assert np.array_equal(np_(ck), np_(ak)) and np.array_equal(np_(cv), np_(av))
    with pytest.raises(ValueError):
        kc.store_kv(vc, k, v, out_k=ck, out_v=cv, capacity=tokens - 1)
    with pytest.raises(ValueError):
        kc.store_kv(vc, k, v, out_k=ck[:-128], out_v=cv, capacity=capacity)
    with pytest.raises(ValueError):
        kc.store_kv(vc, k, v, capacity=capacity)


@pytest.mark.parametrize("fmt", [("turbo3", "turbo3"), ("q8_0", "turbo2")])
def test_layer_prefill_then_decode(fmt):
    """LayerKV.prefill (fp16 prompt) followed by single-token appends: attention over the growing cache against the
    oracle on the same buffers' codes."""
    from test_gpu_attention import assert_close, reference_attention
    B, Hq, Hkv, capacity, prompt = 2, 8, 2, 384, 200
    layer = tqa.LayerKV(tqa.LayerFormat(*fmt), seed=3)
    rng = np.random.default_rng(13)
    k = rng.standard_normal((B * Hkv, prompt + 3, D)).astype(np.float16)
    v = rng.standard_normal((B * Hkv, prompt + 3, D)).astype(np.float16)
    kc, vc = layer.new_cache(B * Hkv, capacity)
    layer.prefill(k[:, :prompt], v[:, :prompt], kc, vc, capacity)
    attn = layer.attention(B, Hq, Hkv, prompt, n_splits=2, capacity=capacity)
    pos = prompt
    for _ in range(3):
        layer.append(k[:, pos:pos + 1], v[:, pos:pos + 1], kc, vc, pos, capacity)
        pos += 1
    q = rng.standard_normal((B, Hq, D)).astype(np.float16)
    attn.set_tokens(pos)
    out = np_(attn(q, kc, vc)).copy()
    ref, _, _ = reference_attention(q, layer.k_codec, layer.v_codec, kc, vc, B, Hq, Hkv, pos, 1 / np.sqrt(D), capacity=capacity,
                                    k_q8=kc if layer.k_codec is None else None, v_q8=vc if layer.v_codec is None else None)
    assert_close(out, ref)


def test_attention_with_the_context_length_on_the_device():
    """tq_attn_params.tokens_dev: the same launch parameters at several context lengths, the length read from device
    memory, against objects built for each length on the host (the split geometry follows the length in the same way,
    so the results are equal bit for bit); lengths above the maximum are clamped to it."""
    tt = L.torch()
    B, Hq, Hkv, cap = 2, 8, 2, 1280
    kc, vc = tqa.TurboCodec(3, seed=42), tqa.TurboCodec(3, seed=542)
    rng = np.random.default_rng(31)
    k = rng.standard_normal((B * Hkv, cap, D)).astype(np.float16)
    v = rng.standard_normal((B * Hkv, cap, D)).astype(np.float16)
    ck, cv = kc.store_kv(vc, k, v)
    q = rng.standard_normal((B, Hq, D)).astype(np.float16)
    bias = tt.from_numpy(rng.standard_normal((B, Hq, cap)).astype(np.float32)).cuda()
    n_dev = tt.zeros(1, dtype=tt.int64, device="cuda")
    moving = tqa.DecodeAttention(kc, vc, B, Hq, Hkv, cap, n_splits=4, capacity=cap, tokens_on_device=n_dev)
    for n in (1, 63, 64, 65, 200, 1000, 1279, 1280):
        n_dev.fill_(n)
        fixed = tqa.DecodeAttention(kc, vc, B, Hq, Hkv, n, n_splits=4, capacity=cap)
        got = np_(moving(q, ck, cv)).copy()
        assert np.array_equal(got, np_(fixed(q, ck, cv))), n
        # with a bias: its rows keep the stride of the maximum length
        got_b = np_(moving(q, ck, cv, bias=bias)).copy()
        want_b = np_(fixed(q, ck, cv, bias=bias[:, :, :n].contiguous()))
        assert np.array_equal(got_b, want_b), n
    n_dev.fill_(5000)
    assert np.array_equal(np_(moving(q, ck, cv)), got)
    with pytest.raises(ValueError):
        tqa.DecodeAttention(kc, vc, B, Hq, Hkv, cap, capacity=cap, tokens_on_device=n_dev, sparse_v_tau=1e-3)


@pytest.mark.parametrize("n_new", [1, 3])
def test_decode_loop_replayed_from_one_hip_graph(n_new):
    """A whole decode step - append at a position held in device memory, advance it, attention over the new length -
    captured once and replayed while the cache grows across a block boundary; every replay against the eager step
    with host positions (bit for bit, cache bytes included), with eager work between the replays."""
    tt = L.torch()
    B, Hq, Hkv, cap, start = 2, 8, 2, 512, 250
    kc, vc = tqa.TurboCodec(3, seed=42), tqa.TurboCodec(3, seed=542)
    rng = np.random.default_rng(6)
    k0 = rng.standard_normal((B * Hkv, start, D)).astype(np.float16)
    v0 = rng.standard_normal((B * Hkv, start, D)).astype(np.float16)
    ck = tt.zeros(tqa.packed_bytes(3, B * Hkv, cap), dtype=tt.uint8, device="cuda")
    cv = tt.zeros_like(ck)
    kc.store_kv(vc, k0, v0, out_k=ck, out_v=cv, capacity=cap)
    ek, ev = ck.clone(), cv.clone()                      # the eager loop's cache
    pos_d = tt.full((1,), start, dtype=tt.int64, device="cuda")
    len_d = tt.full((1,), start, dtype=tt.int64, device="cuda")
    q_s = tt.zeros((B, Hq, D), dtype=tt.float16, device="cuda")
    kn_s = tt.zeros((B * Hkv, n_new, D), dtype=tt.float16, device="cuda")
    vn_s = tt.zeros_like(kn_s)
    attn = tqa.DecodeAttention(kc, vc, B, Hq, Hkv, cap, n_splits=4, capacity=cap, tokens_on_device=len_d)

    def step():
        kc.append_kv(vc, kn_s, vn_s, ck, cv, pos_d, cap)
        pos_d.add_(n_new)
        len_d.add_(n_new)
        return attn(q_s, ck, cv)

    side = tt.cuda.Stream()
    side.wait_stream(tt.cuda.current_stream())
    with tt.cuda.stream(side):
        step()                                           # warm-up outside the capture, then undone
    tt.cuda.current_stream().wait_stream(side)
    ck.copy_(ek)
    cv.copy_(ev)
    pos_d.fill_(start)
    len_d.fill_(start)
    graph = tt.cuda.CUDAGraph()
    with tt.cuda.graph(graph):
        out_g = step()
    ck.copy_(ek)                                         # the capture does not run the kernels; start clean anyway
    cv.copy_(ev)
    pos_d.fill_(start)
    len_d.fill_(start)
    pos = start
    for trial in range(6):                               # 250 -> 256 / 268: crosses the block boundary at 256
        q = tt.from_numpy(rng.standard_normal((B, Hq, D)).astype(np.float16)).cuda()
        kn = tt.from_numpy(rng.standard_normal((B * Hkv, n_new, D)).astype(np.float16)).cuda()
        vn = tt.from_numpy(rng.standard_normal((B * Hkv, n_new, D)).astype(np.float16)).cuda()
        kc.append_kv(vc, kn, vn, ek, ev, pos, cap)
        pos += n_new
        want = tqa.DecodeAttention(kc, vc, B, Hq, Hkv, pos, n_splits=4, capacity=cap)(q, ek, ev).clone()
        tt.cuda.synchronize()
        q_s.copy_(q)
        kn_s.copy_(kn)
        vn_s.copy_(vn)
        graph.replay()
        tt.cuda.synchronize()
        assert int(pos_d.item()) == pos and int(len_d.item()) == pos
        assert tt.equal(ck, ek) and tt.equal(cv, ev), f"cache after replay {trial}"
        assert tt.equal(out_g, want), f"replay {trial}"
    # a position that leaves no room writes nothing
    pos_d.fill_(cap)
    before = ck.clone()
    kc.append_kv(vc, kn_s, vn_s, ck, cv, pos_d, cap)
    assert tt.equal(ck, before)


@pytest.mark.parametrize("fmt", [("q8_0", "turbo2"), ("turbo3", "q8_0"), ("q8_0", "q8_0"), ("turbo4", "turbo3")])
def test_layer_appends_at_a_position_on_the_device(fmt):
    """LayerKV.append with the position in device memory (tq_append_kv_at, tq_append_at, tq_q8_0_append_at) against the
    same appends at host positions: equal caches, at several alignments, and nothing written where there is no room."""
    tt = L.torch()
    n_seqs, cap = 3, 384
    layer = tqa.LayerKV(tqa.LayerFormat(*fmt), seed=5)
    rng = np.random.default_rng(17)
    k = rng.standard_normal((n_seqs, 300, D)).astype(np.float32)
    v = rng.standard_normal((n_seqs, 300, D)).astype(np.float32)
    ak, av = layer.new_cache(n_seqs, cap)
    bk, bv = layer.new_cache(n_seqs, cap)
    pos_d = tt.zeros(1, dtype=tt.int64, device="cuda")
    over = tt.zeros(1, dtype=tt.int32, device="cuda")     # the sticky word a refused position sets
    pos = 0
    for n_new in (100, 27, 1, 1, 130, 1):          # 0 -> 100 -> 127 -> 128 -> 129 -> 259 -> 260
        layer.append(k[:, pos:pos + n_new], v[:, pos:pos + n_new], ak, av, pos, cap)
        pos_d.fill_(pos)
        layer.append(k[:, pos:pos + n_new], v[:, pos:pos + n_new], bk, bv, pos_d, cap, overrun=over)
        pos += n_new
        assert tt.equal(ak, bk) and tt.equal(av, bv), f"after {pos} tokens"
    assert overrun_bits(over) == 0                  # every position so far had room
    pos_d.fill_(cap - 2)                            # the last position with room for two tokens: accepted
    layer.append(k[:, :2], v[:, :2], bk, bv, pos_d, cap, overrun=over)
    layer.append(k[:, :2], v[:, :2], ak, av, cap - 2, cap)
    assert overrun_bits(over) == 0 and tt.equal(ak, bk) and tt.equal(av, bv)
    # no room: nothing written, TQ_OK all the same, and the word says so and keeps saying so
    pos_d.fill_(cap - 1)
    layer.append(k[:, :2], v[:, :2], bk, bv, pos_d, cap)                 # without a word: silent, as before
    assert tt.equal(ak, bk) and tt.equal(av, bv)
    layer.append(k[:, :2], v[:, :2], bk, bv, pos_d, cap, overrun=over)
    assert tt.equal(ak, bk) and tt.equal(av, bv) and overrun_bits(over) == OVERRUN_NO_ROOM
    pos_d.fill_(0)
    layer.append(k[:, :2], v[:, :2], bk, bv, pos_d, cap, overrun=over)   # a good append later does not clear it
    layer.append(k[:, :2], v[:, :2], ak, av, 0, cap)
    assert tt.equal(ak, bk) and tt.equal(av, bv) and overrun_bits(over) == OVERRUN_NO_ROOM
    # a negative position, and a counter full of garbage whose sum with n_new would wrap an int64
    pos_d.fill_(-5)
    layer.append(k[:, :2], v[:, :2], bk, bv, pos_d, cap, overrun=over)
    assert tt.equal(ak, bk) and tt.equal(av, bv) and overrun_bits(over) == OVERRUN_NO_ROOM | OVERRUN_NEGATIVE
    over.zero_()
    pos_d.fill_(2 ** 63 - 1)
    layer.append(k[:, :2], v[:, :2], bk, bv, pos_d, cap, overrun=over)
    assert tt.equal(ak, bk) and tt.equal(av, bv) and overrun_bits(over) == OVERRUN_NO_ROOM
    with pytest.raises(ValueError):
        layer.append(k[:, :2], v[:, :2], bk, bv, pos_d, cap, overrun=tt.zeros(1, dtype=tt.int64, device="cuda"))
    with pytest.raises(ValueError):
        layer.append(k[:, :2], v[:, :2], bk, bv, tt.zeros(1, dtype=tt.int32, device="cuda"), cap)
