"""tq_decode_attention_static (the entry point that allocates nothing: its split partials live in a device
array built into the library) against tq_decode_attention, through the C ABI.  Both run the same kernels, so
the outputs must be bit-identical; the second call is smaller than the first and must not see the first
call's leftovers in the shared workspace."""
import ctypes as C

import numpy as np
import pytest

import tq_oracle as O
import turboquant_plus_amd as tqa
from turboquant_plus_amd import _lib as L

pytestmark = pytest.mark.gpu
D = 128


def run_pair(kc, vc, B, Hq, Hkv, N, n_splits, tau, seed, with_bias):
    tt = L.torch()
    rng = np.random.default_rng(seed)
    k = rng.standard_normal((B * Hkv, N, D)).astype(np.float16)
    v = rng.standard_normal((B * Hkv, N, D)).astype(np.float16)
    q = tt.from_numpy(rng.standard_normal((B, Hq, D)).astype(np.float16)).cuda()
    kp, vp = kc.store(k, kind="k"), vc.store(v, kind="v")
    bias = tt.from_numpy((0.5 * rng.standard_normal((B, Hq, N))).astype(np.float32)).cuda() if with_bias else None
    params = L.TQAttnParams(batch=B, n_q_heads=Hq, n_kv_heads=Hkv, tokens=N, capacity=0, n_splits=n_splits,
                            k_format=L.KFMT_TURBO, v_format=L.KFMT_TURBO, scale=1 / np.sqrt(D), sparse_v_tau=tau)
    ws = tt.empty(int(L.lib().tq_attn_workspace_bytes(C.byref(params))), dtype=tt.uint8, device="cuda")
    out_ws = tt.full((B, Hq, D), float("nan"), dtype=tt.float32, device="cuda")
    out_st = tt.full((B, Hq, D), float("nan"), dtype=tt.float32, device="cuda")
    skip_ws = tt.zeros(2, dtype=tt.int64, device="cuda")
    skip_st = tt.zeros(2, dtype=tt.int64, device="cuda")
    lib, s = L.lib(), L.stream_ptr()
    L.check(lib.tq_decode_attention(kc.handle.h, vc.handle.h, C.byref(params), L.ptr(q), L.TQ_F16, L.ptr(kp), None,
                                    L.ptr(vp), L.ptr(bias), L.ptr(out_ws), L.ptr(skip_ws if tau else None), L.ptr(ws),
                                    ws.numel(), s))
    L.check(lib.tq_decode_attention_static(kc.handle.h, vc.handle.h, C.byref(params), L.ptr(q), L.TQ_F16, L.ptr(kp),
                                           L.ptr(vp), L.ptr(bias), L.ptr(out_st), L.ptr(skip_st if tau else None), s))
    tt.cuda.synchronize()
    assert tt.isfinite(out_st).all()
    assert tt.equal(out_st, out_ws)
    assert tt.equal(skip_st, skip_ws)
    if tau:
        assert int(skip_st[1]) == B * Hq * N
    # and against the oracle, one group
    ki, kg = kc.unpack_codes(kp, B * Hkv, N, kind="k")
    vi, vg = vc.unpack_codes(vp, B * Hkv, N, kind="v")
    k_rot = O.turbo_decode_rotated(ki[0].cpu().numpy(), kg[0].cpu().numpy().astype(np.float64), kc.centroids)
    v_rot = O.turbo_decode_rotated(vi[0].cpu().numpy(), vg[0].cpu().numpy().astype(np.float64), vc.centroids)
    G = Hq // Hkv
    q_rot = O.rotate_fast(q[0, :G].cpu().numpy().astype(np.float64), kc.signs1, kc.signs2, D)
    o, _, _ = O.decode_attention(q_rot, k_rot, v_rot, 1 / np.sqrt(D), n_splits=n_splits, sparse_v_tau=tau,
                                 logit_bias=None if bias is None else bias[0, :G].cpu().numpy().astype(np.float64))
    ref = O.rotate_fast(o, vc.signs1, vc.signs2, D, transpose=True)
    got = out_st[0, :G].cpu().numpy()
    assert np.all(np.abs(got - ref).max(-1) <= 2e-3 * np.abs(ref).max(-1))


def test_static_workspace_entry_point_two_calls_in_a_row():
    kc, vc = tqa.TurboCodec(3, seed=42), tqa.TurboCodec(3, seed=542)
    # a larger call first (64 splits: four workgroups per group, Sparse V with its per-workgroup skip slots) ...
    run_pair(kc, vc, 3, 8, 2, 5000, 64, 1e-3, seed=1, with_bias=True)
    # ... then a smaller one on the same device array: fewer groups, fewer splits, shorter context, dense
    run_pair(kc, vc, 1, 4, 1, 700, 2, 0.0, seed=2, with_bias=False)
    # and Sparse V again on a small shape (skip slots of the first call must not be counted)
    run_pair(kc, vc, 1, 8, 2, 300, 1, 1e-2, seed=3, with_bias=False)


def test_static_workspace_rejects_what_does_not_fit():
    kc, vc = tqa.TurboCodec(3, seed=42), tqa.TurboCodec(3, seed=542)
    tt = L.torch()
    B, Hq, Hkv, N = 64, 32, 8, 64 * 64
    # an odd split count: one wavefront per workgroup, so every split is a partial of its own (512 groups x 63 x 2 KB)
    params = L.TQAttnParams(batch=B, n_q_heads=Hq, n_kv_heads=Hkv, tokens=N, capacity=0, n_splits=63,
                            k_format=L.KFMT_TURBO, v_format=L.KFMT_TURBO, scale=0.1, sparse_v_tau=0.0)
    assert L.lib().tq_attn_workspace_bytes(C.byref(params)) > 16 * 1024 * 1024
    dummy = tt.zeros(4096, dtype=tt.uint8, device="cuda")      # never read: the size check comes first
    rc = L.lib().tq_decode_attention_static(kc.handle.h, vc.handle.h, C.byref(params), L.ptr(dummy), L.TQ_F16,
                                            L.ptr(dummy), L.ptr(dummy), None, L.ptr(dummy), None, L.stream_ptr())
    assert rc == L.ERR_UNSUPPORTED
    assert "built-in workspace" in L.last_error()
