"""GPU tests of the benchmark's measurement probes (libtq_probe.so: tq_probe_stream, tq_probe_flat, tq_probe_mfma_f16) and of
the score tile's store-less mode.  They have no counterpart in the reference: the checks are that the streaming probe
moves exactly the bytes it is asked to, in both access orders, and that the other two run and report."""
import numpy as np
import pytest

import turboquant_plus_amd as tqa
from turboquant_plus_amd import _lib as L
from turboquant_plus_amd import probes
from test_gpu_turbo import np_

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("chunked", [False, True])
@pytest.mark.parametrize("nbytes", [16, 4096 + 16, 3 * 1024 * 1024 + 48])
def test_stream_probe_moves_the_bytes(chunked, nbytes):
    tt = L.torch()
    src = tt.randint(0, 256, (nbytes + 32,), dtype=tt.uint8, device="cuda")
    dst = tt.full((nbytes + 32,), 7, dtype=tt.uint8, device="cuda")
    probes.probe_stream("copy", src[:nbytes], dst[:nbytes], chunked)
    got = np_(dst)
    assert np.array_equal(got[:nbytes], np_(src)[:nbytes])
    assert (got[nbytes:] == 7).all(), "wrote past the end"
    probes.probe_stream("write", None, dst[:nbytes], chunked)
    got = np_(dst).copy()
    assert (got[nbytes:] == 7).all(), "wrote past the end"
    words = got[:nbytes].view(np.uint32).reshape(-1, 4)
    assert (words[:, 1] == 1).all() and (words[:, 2] == 2).all() and (words[:, 3] == 3).all()
    before = np_(src).copy()
    probes.probe_stream("read", src[:nbytes], None, chunked)
    assert np.array_equal(np_(src), before)


def test_stream_probe_rejects_bad_sizes():
    tt = L.torch()
    buf = tt.zeros(64, dtype=tt.uint8, device="cuda")
    with pytest.raises(ValueError):
        probes.probe_stream("copy", buf[:24], buf[32:56])
    with pytest.raises(ValueError):
        probes.probe_stream("write", None, None)


@pytest.mark.parametrize("w64", [0, 13, 17, 64])
def test_flat_probe_touches_exactly_its_share(w64):
    """Every workgroup writes its own write_64ths/64 of 16 KB, back to back with its neighbours', and nothing else;
    what it writes is the xor of the four chunks a lane read with the lane's fill word."""
    tt = L.torch()
    units = 5
    src = tt.randint(0, 256, (units * 16384,), dtype=tt.uint8, device="cuda")
    out_bytes = units * 256 * w64
    dst = tt.full((out_bytes + 64,), 7, dtype=tt.uint8, device="cuda")
    before = np_(src).copy()
    probes.probe_flat(src, dst, units, w64)
    got = np_(dst)
    assert np.array_equal(np_(src), before)
    assert (got[out_bytes:] == 7).all(), "wrote past the end"
    if w64:
        words = before.view(np.uint32).reshape(units, 4, 256, 4)           # [unit][load][lane][word]
        acc = words[:, 0] ^ words[:, 1] ^ words[:, 2] ^ words[:, 3]        # [unit][lane][word]
        acc = acc ^ np.stack([np.arange(256), np.full(256, 1), np.full(256, 2), np.full(256, 3)], axis=1).astype(np.uint32)
        want = np.stack([acc[u][np.arange(16 * w64) % 256] for u in range(units)])
        assert np.array_equal(got[:out_bytes].view(np.uint32).reshape(units, 16 * w64, 4), want)
        # write-only form
        probes.probe_flat(None, dst, units, w64, nontemporal=False)
        got = np_(dst)
        assert (got[out_bytes:] == 7).all()
        assert (got[:out_bytes].view(np.uint32).reshape(-1, 4)[:, 1:] == [1, 2, 3]).all()
    with pytest.raises(ValueError):
        probes.probe_flat(None, None, units, 0)
    with pytest.raises(ValueError):
        probes.probe_flat(src, dst, units + 1, w64)


def test_mfma_probe_reports_its_work():
    tt = L.torch()
    sink = tt.zeros(4, dtype=tt.float32, device="cuda")
    flops = probes.probe_mfma_f16(3, sink)
    tt.cuda.synchronize()
    assert flops == 2048 * 4 * 3 * 8 * 2 * 32 * 32 * 16
    assert float(sink.abs().sum()) == 0.0
    with pytest.raises(ValueError):
        probes.probe_mfma_f16(0, sink)
    with pytest.raises(ValueError):
        probes.probe_mfma_f16(probes.MAX_ITERS + 1, sink)      # a single launch is bounded


def test_score_tile_without_stores_runs():
    tt = L.torch()
    codec = tqa.TurboCodec(3, seed=42, projection="gaussian", projection_seed=2)
    rng = np.random.default_rng(0)
    keys = rng.standard_normal((300, 128)).astype(np.float32)
    qs = rng.standard_normal((70, 128)).astype(np.float16)
    packed, sbits, rn = codec.store_qjl(keys)
    assert codec.score_tile(qs, packed, sbits, rn, 300, store=False) is None
    tt.cuda.synchronize()
    # and the storing call right after it is unaffected
    a = np_(codec.score_tile(qs, packed, sbits, rn, 300))
    b = np_(codec.score_tile(qs, packed, sbits, rn, 300))
    assert np.array_equal(a, b)
