#!/usr/bin/env python3
"""Benchmark of the KV-codec hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one pass of the hot path over one batch of synthetic input:
  * store leg (BASELINE config 2, the `value` of the JSON line): quantise+pack
    one Llama-3-8B-shaped layer, K and V fp16 [8, 32768, 128], 4 outlier
    channels x15 in K, into the turbo4 block format (K and V in one launch);
  * the same leg in turbo3 (the bit width the 70 % target is stated for);
  * decode leg (BASELINE config 3): fused decode attention over turbo3 K/V,
    batch 16, 32 query heads on 8 KV heads, context 32768.
Further legs, each under its own key of the line: config 4 (q8_0-style K, turbo2 V, Sparse V), the config 5 score
tile and QJL store, a boundary layer (q8_0-style K and V), the kernels that rework a packed cache (requantise, export
to and import from the fork's blocks) and the measured peaks of this box (stream probes, fp16 MFMA loop).  The store
leg also times fp32 rows (two fp16 terms per value on the matrix cores), the config-3 decode leg a Sparse V variant and
three small-batch shapes, config 4 its attention-sink bias as a sparse list and as dense rows.
Inputs are resident in HBM before the timed region; every step cycles through
several distinct buffer sets so that the 256 MB Infinity Cache cannot serve
the reads.  Kernel durations come from HIP events recorded on the stream the
kernels are launched on (torch's current stream).

The default warm-up is long on purpose (1000 steps, about 50-90 ms per leg):
when a busy stretch starts after idle time the GPU's power management first
drops the core clock from about 1.93 GHz to about 1.3 GHz and brings it back
over the next 25-30 ms (read in-kernel from the cycle and wall-clock counters),
and a 20-step warm-up times that transient (+15-20 % per step) instead of the
sustained rate a serving loop sees.  When the requested `steps` steps of a leg
take less than 60 ms (e.g. --steps 20), the leg is therefore timed as several
consecutive blocks of exactly `steps` steps, after about 40 ms of further untimed
steps (the transient would otherwise sit in the first blocks and in the wall
figure, which is a mean over all of them), and the median block is reported
(`timed_blocks` in the JSON line says how many, `warmup_steps_run` how many
untimed steps preceded them).

Prints ONE JSON line.  `value` is the algorithmic bytes of the turbo4 store over `ms_per_step`, the wall clock of the
timed steps between two synchronisations; `roofline.achieved` is the same bytes over the kernel's own duration.
`roofline` prices the store kernel against 8 TB/s with
the algorithmic bytes per launch (322 B per vector for turbo4: 256 B fp16 in,
64 B codes, 2 B norm); `cpu_baseline` is the NumPy oracle timed on this box's
host cores over a stated sample of the same workload.
"""
import argparse
import json
import math
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
D = 128
# HBM bytes per launch come from the table "HBM traffic per dispatch" of this profile (rocprofv3 --pmc FETCH_SIZE /
# WRITE_SIZE of this file's run, each scaled by the reading of a 1 GiB device copy).  The table is read at run time;
# a missing file or row gives "traffic": null.  The JSON line names the row next to each figure.
TRAFFIC_FILE = "profiles/bench_all_legs_trace_hbm_sq.txt"
TRAFFIC_ROWS = {"store4": "k_store_kv<4, 4, false, __half>", "store3": "k_store_kv<3, 3, false, __half>",
                "decode3": "k_decode_attn<0, 3, 3, false, true, 1, false, false>"}


def profile_traffic(key):
    """(HBM bytes per launch, where the figure comes from) for one of TRAFFIC_ROWS, from the committed profile's
    traffic table: columns kernel | FETCH KiB | read MB | WRITE KiB | write MB | traffic MB | ..."""
    kernel = TRAFFIC_ROWS[key]
    source = f"{TRAFFIC_FILE}, row {kernel} of the HBM traffic table (recorded by the profiler runs named there, not measured in this run)"
    try:
        in_table = False
        for line in open(os.path.join(ROOT, TRAFFIC_FILE)):
            if line.startswith("== "):
                in_table = line.startswith("== HBM traffic per dispatch")
            elif in_table and line.startswith(kernel):
                cols = line[len(kernel):].split()
                return float(cols[4]) * 1e6, source
    except (OSError, ValueError, IndexError):
        pass
    return None, f"{TRAFFIC_FILE} has no row {kernel}"


METRIC = "KV quantize GB/s + turbo3 decode-attn µs/step @32K ctx, % of HBM roofline"


def synth_kv(torch, heads, tokens, seed, outliers):
    """N(0,1) fp16 [heads, tokens, 128]; `outliers` fixed channels per head scaled x15."""
    g = torch.Generator(device="cuda").manual_seed(seed)
    x = torch.randn((heads, tokens, D), generator=g, device="cuda", dtype=torch.float32)
    if outliers:
        for h in range(heads):
            ch = np.random.default_rng(1000 + h).choice(D, size=outliers, replace=False)
            x[h][:, torch.as_tensor(ch, device="cuda")] *= 15.0
    return x.to(torch.float16)


MIN_TIMED_MS = 60.0   # a leg whose `steps` steps take less than this is timed as several blocks of `steps` steps
PRE_ROLL_MS = 40.0    # ... after this much further untimed work, which carries the launch stream past the clock transient


def time_steps(torch, step, steps, warmup, info=None):
    """(wall ms per step with sync brackets, event ms per step on the launch stream).

    Exactly `steps` steps are timed between two events / two synchronisations.  When that stretch is shorter
    than MIN_TIMED_MS it sits inside the clock transient that follows idle time (see the module text), so the
    measurement is repeated as consecutive blocks of `steps` steps, MIN_TIMED_MS of timed work in all (at
    least 5 blocks), and the block with the median event time is reported; the wall figure is the mean over the
    whole stretch.  info["timed_blocks"] says how many blocks were timed."""
    for i in range(warmup):
        step(i)
    torch.cuda.synchronize()

    def run_blocks(n_blocks, first):
        """n_blocks consecutive blocks of `steps` steps with an event between blocks and no host wait in between
        (a synchronisation per block would let the clock fall back during the gap)."""
        ev = [torch.cuda.Event(enable_timing=True) for _ in range(n_blocks + 1)]
        t0 = time.perf_counter()
        ev[0].record()
        for b in range(n_blocks):
            for i in range(steps):
                step(first + b * steps + i)
            ev[b + 1].record()
        torch.cuda.synchronize()
        wall = (time.perf_counter() - t0) * 1e3
        return [ev[b].elapsed_time(ev[b + 1]) for b in range(n_blocks)], wall

    times, wall = run_blocks(1, warmup)
    n_blocks = 1
    extra = 0
    if times[0] < MIN_TIMED_MS:
        n_blocks = int(min(400, max(5, math.ceil(MIN_TIMED_MS / max(times[0], 1e-3)))))
        # the transient also sits in the first blocks of such a stretch and would raise the wall figure, which is a mean
        # over all blocks: PRE_ROLL_MS of further untimed steps first (what the default's 1000 warm-up steps amount to)
        extra = int(math.ceil(PRE_ROLL_MS / max(times[0] / steps, 1e-4)))
        for i in range(extra):
            step(warmup + steps + i)
        torch.cuda.synchronize()
        times, wall = run_blocks(n_blocks, warmup + steps + extra)
    if info is not None:
        info["timed_blocks"] = n_blocks
        info["warmup_steps_run"] = warmup + (steps + extra if n_blocks > 1 else 0)
    return wall / (n_blocks * steps), sorted(times)[n_blocks // 2] / steps


def measured_peaks_leg(torch, tqa, steps, warmup):
    """What this box sustains on plain streaming kernels (1 GiB, two buffer sets) and on back-to-back fp16
    MFMAs, timed like the legs below; set beside the published peaks the fractions are quoted against."""
    from turboquant_plus_amd import probes
    n = 1 << 30
    bufs = [torch.empty(n, dtype=torch.uint8, device="cuda") for _ in range(4)]
    for b in bufs:
        b.zero_()
    out = {"bytes_per_launch": n}
    reps, warm = max(20, steps // 10), max(10, warmup // 10)
    for mode in ("read", "write", "copy", "read_nt", "write_nt", "copy_nt"):   # _nt: non-temporal hint on every access
        best = 0.0
        for chunked in (False, True):   # lanes striding over the whole buffer, or one contiguous slice per workgroup
            def step(i):
                src, dst = bufs[2 * (i % 2)], bufs[2 * (i % 2) + 1]
                probes.probe_stream(mode, None if mode.startswith("write") else src, None if mode.startswith("read") else dst, chunked)
            _, ev_ms = time_steps(torch, step, reps, warm)
            moved = n * (2 if mode.startswith("copy") else 1)
            best = max(best, moved / (ev_ms * 1e-3) / 1e9)
        out[f"hbm_{mode}_gbs"] = best   # the better of the two access orders
    # short-lived workgroups in dispatch order (one compact window moving through memory): the read/write mixes of the
    # fused K+V store at config 2 (128 MiB of fp16 rows in, 13/64 or 17/64 of that out) and the fp32 logits of config 5
    # (512 MiB written) as bare traffic, the floor a kernel with that traffic and nothing else would reach on this box
    flat = {}
    units = (128 << 20) // 16384
    for name, w64 in (("store_mix_turbo3", 13), ("store_mix_turbo4", 17), ("read_128MiB", 0)):
        def step(i, w64=w64):
            probes.probe_flat(bufs[i % 4], bufs[(i + 1) % 4][(512 << 20):], units, w64)
        _, ev_ms = time_steps(torch, step, steps, warmup)   # short launches: as many as the store legs, past the clock transient
        moved = units * (16384 + 256 * w64)
        flat[name] = {"us": ev_ms * 1e3, "gbs": moved / (ev_ms * 1e-3) / 1e9}

    def wstep(i):
        probes.probe_flat(None, bufs[i % 4], (512 << 20) // 16384, 64)
    _, ev_ms = time_steps(torch, wstep, max(reps, steps // 4), max(warm, warmup // 4))
    flat["write_512MiB"] = {"us": ev_ms * 1e3, "gbs": (512 << 20) / (ev_ms * 1e-3) / 1e9}
    out["flat"] = flat
    del bufs
    sink = torch.zeros(4, dtype=torch.float32, device="cuda")
    flops = [0]

    def mstep(i):
        flops[0] = probes.probe_mfma_f16(2000, sink)
    _, ev_ms = time_steps(torch, mstep, reps, warm)
    out["mfma_f16_tflops"] = flops[0] / (ev_ms * 1e-3) / 1e12
    out["published"] = {"hbm_gbs": HBM_PEAK_GBS, "mfma_f16_tflops": 2500.0}
    return out


def store_leg(torch, tqa, bits, steps, warmup, n_sets=4, several_streams=False):
    heads, tokens = 8, 32768
    codec_k, codec_v = tqa.TurboCodec(bits, seed=42), tqa.TurboCodec(bits, seed=542)
    sets = []
    for s in range(n_sets):
        k = synth_kv(torch, heads, tokens, 10 + s, outliers=4)
        v = synth_kv(torch, heads, tokens, 20 + s, outliers=0)
        kp = torch.empty(tqa.packed_bytes(bits, heads, tokens), dtype=torch.uint8, device="cuda")
        vp = torch.empty_like(kp)
        sets.append((k, v, kp, vp))

    def step(i):
        k, v, kp, vp = sets[i % n_sets]
        codec_k.store_kv(codec_v, k, v, out_k=kp, out_v=vp)      # one launch for the layer's K and V

    info = {}
    wall_ms, ev_ms = time_steps(torch, step, steps, warmup, info)
    n_vec = 2 * heads * tokens
    bytes_per_vec = 256 + 16 * bits + 2
    algo = n_vec * bytes_per_vec
    launch_us = ev_ms * 1e3                          # one launch (K and V) per step
    gbs = algo / (launch_us * 1e-6) / 1e9
    # consecutive layers issued on several streams (--several-streams; what a serving loop that stores a layer's K and V
    # per step can do: layers are independent, so one launch's tail overlaps the next one's start); wall clock over the
    # whole loop.  Off by default: its launches overlap, which would blur the kernel's row in a trace of the default run.
    two_us = None
    if several_streams:
        # (the C entry point is called with prepared arguments, so that the host's share of a call stays well below a launch)
        import ctypes
        from turboquant_plus_amd import _lib as L
        streams = [torch.cuda.Stream() for _ in range(4)]   # four: one per hardware queue of the process
        sp = [ctypes.c_void_p(st.cuda_stream) for st in streams]
        fn, hk, hv, code = L.lib().tq_store_kv, codec_k.handle.h, codec_v.handle.h, L.dtype_code(sets[0][0])
        prepared = [tuple(L.ptr(t) for t in st) for st in sets]

        def run_two(n):
            for i in range(n):
                pk_, pv_, pkp, pvp = prepared[i % n_sets]
                if fn(hk, hv, pk_, pv_, heads, tokens, code, pkp, pvp, sp[i % 4]):
                    raise RuntimeError(L.last_error())
        run_two(warmup)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        run_two(max(steps, 1000))
        torch.cuda.synchronize()
        two_us = (time.perf_counter() - t0) / max(steps, 1000) * 1e6
    # the same tensors as the prompt of a cache laid out for 40 960 tokens per sequence (tq_store_kv_cache)
    cap = tokens + 8192
    caches = [(torch.empty(tqa.packed_bytes(bits, heads, cap), dtype=torch.uint8, device="cuda"),
               torch.empty(tqa.packed_bytes(bits, heads, cap), dtype=torch.uint8, device="cuda")) for _ in range(2)]

    def pstep(i):
        k_, v_, _, _ = sets[i % n_sets]
        ck_, cv_ = caches[i % 2]
        codec_k.store_kv(codec_v, k_, v_, out_k=ck_, out_v=cv_, capacity=cap)
    _, pev_ms = time_steps(torch, pstep, steps, warmup)
    del caches
    # round-trip error of the last set
    k, v, kp, vp = sets[0]
    rec = codec_k.load(kp, heads, tokens, kind="k", domain="original")
    rel = float((((rec - k.float()) ** 2).sum(-1) / (k.float() ** 2).sum(-1)).mean())
    del rec
    # decompress (the way back): K and V of the layer to fp16 in the original domain, one launch per step
    outs = [(torch.empty_like(k), torch.empty_like(v)) for _ in range(2)]

    def lstep(i):
        _, _, kp_i, vp_i = sets[i % n_sets]
        ok, ov = outs[i % 2]
        codec_k.load_kv(codec_v, kp_i, vp_i, heads, tokens, out_k=ok, out_v=ov)
    _, lev_ms = time_steps(torch, lstep, steps, warmup)
    load_algo = n_vec * (16 * bits + 2 + 256)
    # fp32 rows (the reference's input type; config 1's path): the same K and V tensors as float32 through tq_store_kv,
    # which runs the matrix-core kernels on two fp16 terms per value, one launch per tensor; and K alone
    f32 = None
    if bits == 3:
        sets32 = [(k_.float(), v_.float(), kp_, vp_) for (k_, v_, kp_, vp_) in sets[:2]]

        def fstep(i):
            k_, v_, kp_, vp_ = sets32[i % 2]
            codec_k.store_kv(codec_v, k_, v_, out_k=kp_, out_v=vp_)

        def fkstep(i):
            k_, _, kp_, _ = sets32[i % 2]
            codec_k.store(k_, kind="k", out=kp_)
        def fvstep(i):
            _, v_, _, vp_ = sets32[i % 2]
            codec_v.store(v_, kind="v", out=vp_)
        _, fev_ms = time_steps(torch, fstep, steps, warmup)
        _, fkev_ms = time_steps(torch, fkstep, steps, warmup)
        _, fvev_ms = time_steps(torch, fvstep, steps, warmup)
        f_algo = n_vec * (512 + 16 * bits + 2)
        f32 = {"what": "K and V as float32 rows (512 B per vector in), one launch (k_store_kv<float>); k_alone / v_alone: the single-tensor kernels",
               "us_per_step": fev_ms * 1e3, "algorithmic_bytes_per_step": f_algo, "gbs": f_algo / (fev_ms * 1e-3) / 1e9,
               "frac": f_algo / (fev_ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
               "k_alone": {"us_per_launch": fkev_ms * 1e3, "gbs": f_algo / 2 / (fkev_ms * 1e-3) / 1e9,
                           "frac": f_algo / 2 / (fkev_ms * 1e-3) / 1e9 / HBM_PEAK_GBS},
               "v_alone": {"us_per_launch": fvev_ms * 1e3, "gbs": f_algo / 2 / (fvev_ms * 1e-3) / 1e9,
                           "frac": f_algo / 2 / (fvev_ms * 1e-3) / 1e9 / HBM_PEAK_GBS}}
        del sets32
        # float64 rows (the reference's own dtype): the butterfly kernel k_store, one launch per tensor; K alone
        k64 = sets[0][0].double()
        kp64 = sets[0][2]

        def dstep(i):
            codec_k.store(k64, kind="k", out=kp64)
        _, dev_ms = time_steps(torch, dstep, max(steps // 2, 1), warmup)
        d_algo = n_vec // 2 * (1024 + 16 * bits + 2)
        f32["f64_rows_k_alone"] = {"what": "the K tensor as float64 rows (1024 B per vector in) through the butterfly kernel (k_store<double>)",
                                   "us_per_launch": dev_ms * 1e3, "algorithmic_bytes_per_launch": d_algo,
                                   "gbs": d_algo / (dev_ms * 1e-3) / 1e9, "frac": d_algo / (dev_ms * 1e-3) / 1e9 / HBM_PEAK_GBS}
        codec_k.store(sets[0][0], kind="k", out=kp64)      # the set's packed K as the fp16 rows give it
        del k64
    return {
        "workload": f"turbo{bits} store, K+V fp16 [8,32768,128], 4 K outlier channels x15, block 128",
        "ms_per_step": wall_ms, "event_ms_per_step": ev_ms, "kernel_us": launch_us,
        "algorithmic_bytes_per_launch": algo, "gbs": gbs, "frac": gbs / HBM_PEAK_GBS,
        "roundtrip_rel_mse_k": rel, "buffer_sets": n_sets, "timed_blocks": info["timed_blocks"],
        "warmup_steps_run": info["warmup_steps_run"],
        "prefill_into_cache": {"us_per_launch": pev_ms * 1e3, "capacity": cap,
                               "what": "the same K and V as the prompt of caches laid out for `capacity` tokens per sequence"},
        "several_streams": None if two_us is None else {
            "streams": 4, "us_per_launch": two_us, "gbs": algo / (two_us * 1e-6) / 1e9, "frac": algo / (two_us * 1e-6) / 1e9 / HBM_PEAK_GBS,
            "what": "the same launches issued round-robin on four streams, wall clock per launch; not the roofline figure"},
        "fp32_rows": f32,
        "decompress": {"us_per_step": lev_ms * 1e3, "launches_per_step": 1, "io": "codes + fp16 norm in, fp16 out",
                       "gbs": load_algo / (lev_ms * 1e-3) / 1e9, "frac": load_algo / (lev_ms * 1e-3) / 1e9 / HBM_PEAK_GBS},
    }


def decode_leg(torch, tqa, steps, warmup, n_sets=2, small_batches=True):
    B, Hq, Hkv, N, bits = 16, 32, 8, 32768, 3
    kc, vc = tqa.TurboCodec(bits, seed=42), tqa.TurboCodec(bits, seed=542)
    sets = []
    for s in range(n_sets):
        kp = torch.empty(tqa.packed_bytes(bits, B * Hkv, N), dtype=torch.uint8, device="cuda")
        vp = torch.empty_like(kp)
        per = kp.numel() // B
        for b in range(B):                            # generated as in the store config, per sequence
            k = synth_kv(torch, Hkv, N, 100 + 16 * s + b, outliers=4)
            v = synth_kv(torch, Hkv, N, 200 + 16 * s + b, outliers=0)
            kc.store_kv(vc, k, v, out_k=kp[b * per:(b + 1) * per], out_v=vp[b * per:(b + 1) * per])   # as a prefill does
        g = torch.Generator(device="cuda").manual_seed(300 + s)
        q = torch.randn((B, Hq, D), generator=g, device="cuda").to(torch.float16)
        sets.append((q, kp, vp))
    attn = tqa.DecodeAttention(kc, vc, B, Hq, Hkv, N)

    def step(i):
        q, kp, vp = sets[i % n_sets]
        attn(q, kp, vp)

    info = {}
    wall_ms, ev_ms = time_steps(torch, step, steps, warmup, info)
    algo = 2 * B * Hkv * N * 50
    us = ev_ms * 1e3
    gbs = algo / (us * 1e-6) / 1e9

    # the same cache under eight query heads per KV head (64 query heads): one pass of eight heads over the K/V
    g8 = torch.Generator(device="cuda").manual_seed(301)
    q64 = torch.randn((B, 2 * Hq, D), generator=g8, device="cuda").to(torch.float16)
    attn8 = tqa.DecodeAttention(kc, vc, B, 2 * Hq, Hkv, N)
    _, ev8_ms = time_steps(torch, lambda i: attn8(q64, sets[i % n_sets][1], sets[i % n_sets][2]), steps, warmup)

    # heads of 256 dims: the same buffers read as 16 384 tokens of two rows each (the same bytes per step)
    g2 = torch.Generator(device="cuda").manual_seed(302)
    q256 = torch.randn((B, Hq, 2 * D), generator=g2, device="cuda").to(torch.float16)
    attn256 = tqa.DecodeAttention(kc, vc, B, Hq, Hkv, N // 2, head_dim=256)
    _, ev256_ms = time_steps(torch, lambda i: attn256(q256, sets[i % n_sets][1], sets[i % n_sets][2]), steps, warmup)

    # Sparse V on this cache (turbo3 K and V: V is half of the bytes): the benchmark's queries and queries scaled x16
    # (peaked attention), with the skip rate the kernel reports
    sparse_v = {}
    for name, qscale in (("bench_queries", 1.0), ("peaked_queries_x16", 16.0)):
        qs_ = [(st[0].float() * qscale).to(torch.float16) for st in sets]
        dn = tqa.DecodeAttention(kc, vc, B, Hq, Hkv, N)
        sp = tqa.DecodeAttention(kc, vc, B, Hq, Hkv, N, sparse_v_tau=1e-6)
        _, d_ms = time_steps(torch, lambda i: dn(qs_[i % n_sets], sets[i % n_sets][1], sets[i % n_sets][2]), steps, warmup)
        _, s_ms = time_steps(torch, lambda i: sp(qs_[i % n_sets], sets[i % n_sets][1], sets[i % n_sets][2]), steps, warmup)
        sparse_v[name] = {"dense_us_per_step": d_ms * 1e3, "sparse_v_us_per_step": s_ms * 1e3, "tau": 1e-6,
                          "skip_rate": sp.skip_rate()}
        del dn, sp

    # small batches on the same kind of cache: few (batch, kv head) groups, so the context splits must fill the chip
    small = {}
    for name, b_, n_ in (("B1_ctx32768", 1, N), ("B4_ctx32768", 4, N), ("B256_ctx2048", 256, 2048)) if small_batches else ():
        per_seq = tqa.packed_bytes(bits, Hkv, n_)
        if b_ * per_seq <= sets[0][1].numel():
            kp_, vp_ = sets[0][1][:b_ * per_seq], sets[0][2][:b_ * per_seq]     # any valid codes do for timing
        else:
            kp_ = sets[0][1].repeat(-(-b_ * per_seq // sets[0][1].numel()))[:b_ * per_seq]
            vp_ = sets[0][2].repeat(-(-b_ * per_seq // sets[0][2].numel()))[:b_ * per_seq]
        gq = torch.Generator(device="cuda").manual_seed(400 + b_)
        qb = torch.randn((b_, Hq, D), generator=gq, device="cuda").to(torch.float16)
        at = tqa.DecodeAttention(kc, vc, b_, Hq, Hkv, n_)
        _, sm_ms = time_steps(torch, lambda i: at(qb, kp_, vp_), steps, warmup)
        sm_algo = 2 * b_ * Hkv * n_ * 50
        small[name] = {"us_per_step": sm_ms * 1e3, "n_splits": at.params.n_splits, "algorithmic_bytes_per_step": sm_algo,
                       "gbs": sm_algo / (sm_ms * 1e-3) / 1e9, "frac": sm_algo / (sm_ms * 1e-3) / 1e9 / HBM_PEAK_GBS}
        del at, kp_, vp_

    # a whole serving step: append this step's K and V token of every sequence (the last position of the
    # cache is rewritten each time), then attention; launched one by one and replayed from one HIP graph
    g = torch.Generator(device="cuda").manual_seed(77)
    k_new = torch.randn((B * Hkv, 1, D), generator=g, device="cuda").to(torch.float16)
    v_new = torch.randn((B * Hkv, 1, D), generator=g, device="cuda").to(torch.float16)

    def serving_step(i):
        q, kp, vp = sets[i % n_sets]
        kc.append_kv(vc, k_new, v_new, kp, vp, N - 1, N)
        attn(q, kp, vp)

    _, serve_ms = time_steps(torch, serving_step, steps, warmup)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        serving_step(0)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for i in range(n_sets):
            serving_step(i)
    _, graph_ms = time_steps(torch, lambda i: graph.replay(), max(1, steps // n_sets), max(1, warmup // n_sets))
    return {
        "workload": "fused decode attention, turbo3 K/V, B16 Hq32 Hkv8 d128 ctx 32768, queries rotated in-step",
        "us_per_step": us, "wall_us_per_step": wall_ms * 1e3, "n_splits": attn.params.n_splits,
        "timed_blocks": info["timed_blocks"], "warmup_steps_run": info["warmup_steps_run"],
        "roofline": {"bound": "hbm", "achieved": gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": gbs / HBM_PEAK_GBS,
                     "traffic": profile_traffic("decode3")[0], "traffic_source": profile_traffic("decode3")[1],
                     "algorithmic_bytes_per_step": algo,
                     "kernel": "k_decode_attn<turbo3,turbo3> (one launch: the last workgroup of a group merges the partials)"},
        "buffer_sets": n_sets,
        "gqa8": {"workload": "the same cache, 64 query heads on 8 KV heads (eight heads per pass over K/V)",
                 "us_per_step": ev8_ms * 1e3, "n_splits": attn8.params.n_splits,
                 "frac": algo / (ev8_ms * 1e-3) / 1e9 / HBM_PEAK_GBS},
        "head_dim_256": {"workload": "the same buffers as 16384 tokens of 256 dims (two 128-value rows per token), 32 query heads on 8 KV heads",
                         "us_per_step": ev256_ms * 1e3, "n_splits": attn256.params.n_splits,
                         "frac": algo / (ev256_ms * 1e-3) / 1e9 / HBM_PEAK_GBS},
        "sparse_v": sparse_v, "small_batches": small,
        "serving_step": {"workload": "tq_append_kv of one token per sequence + decode attention",
                         "us_per_step": serve_ms * 1e3, "us_per_step_hip_graph": graph_ms * 1e3 / n_sets},
    }


def asym_decode_leg(torch, tqa, steps, warmup):
    """BASELINE config 4: K q8_0-style (not rotated), V turbo2, B4 Hq32 Hkv8 ctx 131072, +6 logit bias
    on 64 random key positions per head (given as an additive fp32 bias input), Sparse V tau 1e-6."""
    B, Hq, Hkv, N = 4, 32, 8, 131072
    vc = tqa.TurboCodec(2, seed=542)
    kq = torch.empty(B * Hkv * (N // 128) * 128 * 136, dtype=torch.uint8, device="cuda")
    vp = torch.empty(tqa.packed_bytes(2, B * Hkv, N), dtype=torch.uint8, device="cuda")
    perk, perv = kq.numel() // (B * Hkv), vp.numel() // (B * Hkv)
    for s in range(B * Hkv):                         # one (sequence, kv head) at a time keeps peak memory low
        k = synth_kv(torch, 1, N, 400 + s, outliers=4)
        v = synth_kv(torch, 1, N, 500 + s, outliers=0)
        kq[s * perk:(s + 1) * perk] = tqa.q8_0_store(k)[0]
        vc.store(v, kind="v", out=vp[s * perv:(s + 1) * perv])
    g = torch.Generator(device="cuda").manual_seed(7)
    q = torch.randn((B, Hq, D), generator=g, device="cuda").to(torch.float16)
    bias = torch.zeros((B, Hq, N), dtype=torch.float32, device="cuda")
    pos = torch.stack([torch.randperm(N, generator=g, device="cuda")[:64] for _ in range(B * Hq)]).view(B, Hq, 64)
    bias.scatter_(2, pos, 6.0)
    # fraction of (batch, q-head, position) whose final softmax weight is below tau (the definition of the
    # reference's scripts/measure_skip_rate.py:69-74), from the stored K in fp32; and, with the kernel's own
    # predicate restated in torch, the fraction of 64-token V rows the kernel does not fetch: it drops a tile's
    # PV work when all 4 heads x 64 weights are below tau against the running maximum of the split, requests the
    # next tile's V row ahead only after a tile that was not dropped, and fetches on demand otherwise - so a row
    # stays unfetched when its tile and the tile before it are both dropped (never the first tile of a split).
    def cache_stats(qq, n_splits):
        below, rows_saved, scale = 0, 0, 1.0 / math.sqrt(D)
        tiles_per_split = -(-(N // 64) // n_splits)
        for s in range(B * Hkv):
            qi, sc = tqa.q8_0_unpack(kq[s * perk:(s + 1) * perk], 1, N)
            kd = (qi.view(N, 4, 32).float() * sc.view(N, 4, 1)).view(N, D)
            b, h = divmod(s, Hkv)
            logit = qq[b, 4 * h:4 * h + 4].float() @ kd.t() * scale + bias[b, 4 * h:4 * h + 4]
            below += int((torch.softmax(logit, dim=-1) < 1e-6).sum())
            lt = logit.view(4, N // 64 // tiles_per_split, tiles_per_split, 64)      # [head, split, tile, token]
            run_max = torch.cummax(lt.amax(dim=-1), dim=-1).values                   # running maximum incl. the tile
            dropped = ((lt - run_max[..., None]).exp() < 1e-6).all(dim=-1).all(dim=0)  # [split, tile]
            rows_saved += int((dropped[:, 1:] & dropped[:, :-1]).sum())
            del qi, sc, kd, logit, lt
        return below / float(B * Hq * N), rows_saved / float(B * Hkv * (N // 64))
    out = {}
    q_peaked = (q.float() * 16.0).to(torch.float16)  # a second input for Sparse V: logits 16 x as spread, few tiles matter
    # the sharpening bias as per-head (position, value) lists: 64 entries per head instead of a dense fp32 row per head
    sparse_bias = tqa.sparse_bias_from_dense(bias, max_entries=64)
    for name, tau, qq, as_rows in (("dense", 0.0, q, False), ("dense_bias_as_rows", 0.0, q, True), ("sparse_v", 1e-6, q, False),
                                   ("sparse_v_peaked_queries", 1e-6, q_peaked, False)):
        attn = tqa.DecodeAttention(None, vc, B, Hq, Hkv, N, sparse_v_tau=tau)
        if as_rows:
            wall_ms, ev_ms = time_steps(torch, lambda i: attn(qq, kq, vp, bias=bias), steps, warmup)
        else:
            wall_ms, ev_ms = time_steps(torch, lambda i: attn(qq, kq, vp, sparse_bias=sparse_bias), steps, warmup)
        skip = attn.skip_rate() if tau else 0.0
        algo = B * Hkv * N * (136 + 34)               # dense bytes: the roofline figure of every variant
        us = ev_ms * 1e3
        out[name] = {"us_per_step": us, "skip_rate": skip, "n_splits": attn.params.n_splits,
                     "achieved_gbs": algo / (us * 1e-6) / 1e9, "frac": algo / (us * 1e-6) / 1e9 / HBM_PEAK_GBS}
        if tau:
            final_weight_skip, rows_saved = cache_stats(qq, attn.params.n_splits)
            # the kernel tests exp(logit - running maximum of its split), without the softmax denominator
            out[name]["skip_rate_final_weight"] = final_weight_skip
            out[name]["v_rows_not_fetched"] = rows_saved
            out[name]["bytes_required"] = B * Hkv * N * (136 + (1.0 - rows_saved) * 34)
    out["workload"] = ("decode attention, K q8_0-style + V turbo2, B4 Hq32 Hkv8 ctx 131072, +6 bias on 64 key "
                       "positions per head as 64 (position, value) entries per head (dense_bias_as_rows: the same bias as a dense "
                       "fp32 row per head, 67 MB of input, not counted), Sparse V tau 1e-6; "
                       "sparse_v_peaked_queries: the same cache with the queries scaled x16; skip_rate = (query, position) "
                       "pairs whose weight the kernel dropped, v_rows_not_fetched = fraction of 64-token V rows it never "
                       "requested (whole tiles only), bytes_required = K + the V rows it did request")
    out["algorithmic_bytes_per_step"] = B * Hkv * N * 170
    return out


def score_tile_leg(torch, tqa, steps, warmup):
    """BASELINE config 5: 65536 keys as 3-bit codes + QJL sketch (Gaussian projection, seed 2), 2048 fp16
    queries -> 2048 x 65536 logits through the K=256 MFMA contraction."""
    nk, nq = 65536, 2048
    g = torch.Generator(device="cuda").manual_seed(11)
    keys = torch.randn((nk, D), generator=g, device="cuda", dtype=torch.float32)
    qs = torch.randn((nq, D), generator=g, device="cuda").to(torch.float16)
    codec = tqa.TurboCodec(3, seed=42, projection="gaussian", projection_seed=2)
    packed, sbits, rn = codec.store_qjl(keys)
    out = {"workload": "TurboQuant estimator tile, 65536 keys (3-bit + QJL, gaussian S seed 2) x 2048 fp16 queries"}
    _, q_ms = time_steps(torch, lambda i: codec.store_qjl(keys), max(5, steps // 20), max(2, warmup // 20))
    out["qjl_store"] = {"us_per_call": q_ms * 1e3, "keys_per_s": nk / (q_ms * 1e-3),
                        "what": "codes + corrected norm + residual norm + 128 sign bits per key; float64 arithmetic, the sign "
                                "sketch on the fp16 matrix cores with an error bound and a float64 second pass"}
    flops = 2.0 * nq * nk * 256
    for name, dt in (("fp32_logits", torch.float32), ("fp16_logits", torch.float16)):
        logits = None

        def step(i):
            nonlocal logits
            logits = codec.score_tile(qs, packed, sbits, rn, nk, out_dtype=dt)
        wall_ms, ev_ms = time_steps(torch, step, max(5, steps // 10), max(2, warmup // 10))
        out[name] = {"us_per_call": ev_ms * 1e3, "mfma_tflops": flops / (ev_ms * 1e-3) / 1e12,
                     "mfma_frac_of_2500": flops / (ev_ms * 1e-3) / 2.5e15,
                     "logit_store_gbs": logits.numel() * logits.element_size() / (ev_ms * 1e-3) / 1e9}
        if dt == torch.float32:
            _, dry_ms = time_steps(torch, lambda i: codec.score_tile(qs, packed, sbits, rn, nk, out_dtype=dt, store=False),
                                   max(5, steps // 10), max(2, warmup // 10))
            out["no_store"] = {"us_per_call": dry_ms * 1e3, "mfma_tflops": flops / (dry_ms * 1e-3) / 1e12,
                               "mfma_frac_of_2500": flops / (dry_ms * 1e-3) / 2.5e15}
            exact = qs[:256].float() @ keys.t()
            err = logits[:256] - exact
            out["estimator_bias"] = float(err.mean())
            out["estimator_rms_error"] = float(err.pow(2).mean().sqrt())
            out["exact_rms"] = float(exact.pow(2).mean().sqrt())
    return out


def cpu_baseline(bits):
    """The NumPy oracle on a bounded sample of the store workload: one head of K
    and one head of V (2 x 32768 vectors), encode + pack, float64."""
    sys.path.insert(0, os.path.join(ROOT, "oracle"))
    import tq_oracle as O
    try:
        from threadpoolctl import threadpool_info
        blas_threads = max([p.get("num_threads", 1) for p in threadpool_info()] or [1])
    except Exception:
        blas_threads = None
    rng = np.random.default_rng(0)
    n = 32768
    k = rng.standard_normal((n, D)).astype(np.float16)
    v = rng.standard_normal((n, D)).astype(np.float16)
    s1, s2, _ = O.sign_diagonals(D, np.random.default_rng(42))
    cent = O.centroids_for(bits, D)
    passes, n_samples = 6, 5                          # a sample = 6 passes over one head of K and one of V (about 2 s)
    times = []
    for _ in range(n_samples):
        t0 = time.perf_counter()
        for _ in range(passes):
            for x, kind in ((k, "k"), (v, "v")):
                idx, g, _ = O.turbo_encode(x, s1, s2, cent)
                O.layout_pack(idx, g, bits, kind)
        times.append(time.perf_counter() - t0)
    dt = sorted(times)[n_samples // 2]
    algo = passes * 2 * n * (256 + 16 * bits + 2)
    # attention leg: one (batch, kv head) group of config 3, decompress -> softmax -> PV
    q = rng.standard_normal((4, D))
    idx, g, _ = O.turbo_encode(k, s1, s2, cent)
    vi, vg, _ = O.turbo_encode(v, s1, s2, cent)
    atimes = []
    for _ in range(n_samples):
        t0 = time.perf_counter()
        kr = O.turbo_decode_rotated(idx, g, cent)
        vr = O.turbo_decode_rotated(vi, vg, cent)
        O.decode_attention(O.rotate_fast(q, s1, s2, D), kr, vr, 1 / np.sqrt(D))
        atimes.append(time.perf_counter() - t0)
    dta = sorted(atimes)[n_samples // 2]
    return ({"value": algo / dt / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
             "sample": f"NumPy oracle turbo{bits} encode+pack of {passes} x 2 x 32768 fp16 vectors (one head of K and one of V "
                       f"of config 2, {passes} passes = 3/4 of the layer), median of {n_samples} such samples "
                       f"({dt:.2f} s; min {min(times):.2f}, max {max(times):.2f}), single-threaded NumPy (no BLAS on this path)",
             "host_cpus": os.cpu_count()},
            {"value": dta * 128 * 1e6, "unit": "µs/step", "cores": blas_threads or 1, "kind": "port",
             "sample": f"NumPy oracle decompress->softmax->PV for 1 of 128 (batch, kv-head) groups at ctx 32768 "
                       f"(median of {n_samples} samples: {dta * 1e3:.1f} ms; min {min(atimes) * 1e3:.1f}, max {max(atimes) * 1e3:.1f}), "
                       f"extrapolated x128", "host_cpus": os.cpu_count()})


def boundary_layer_leg(torch, tqa, steps, warmup):
    """A boundary layer of the fork's layer-adaptive modes (K and V kept as q8_0-style rows) at the config-3
    shape: the V store of a prefill and the decode step."""
    B, Hq, Hkv, N = 16, 32, 8, 32768
    per = N * 136
    kq = torch.empty(B * Hkv * per, dtype=torch.uint8, device="cuda")
    vq = torch.empty_like(kq)
    vsets = []
    for b in range(B):
        k = synth_kv(torch, Hkv, N, 600 + b, outliers=4)
        v = synth_kv(torch, Hkv, N, 700 + b, outliers=0)
        kq[b * Hkv * per:(b + 1) * Hkv * per] = tqa.q8_0_store(k)[0]
        vq[b * Hkv * per:(b + 1) * Hkv * per] = tqa.q8_0_store(v, kind="v")[0]
        if b < 4:
            vsets.append(v)
    g = torch.Generator(device="cuda").manual_seed(9)
    q = torch.randn((B, Hq, D), generator=g, device="cuda").to(torch.float16)
    attn = tqa.DecodeAttention(None, None, B, Hq, Hkv, N)
    _, ev_ms = time_steps(torch, lambda i: attn(q, kq, vq), steps, warmup)
    algo = 2 * B * Hkv * per
    us = ev_ms * 1e3
    _, st_ms = time_steps(torch, lambda i: tqa.q8_0_store(vsets[i % 4], kind="v"), steps, warmup)
    st_bytes = Hkv * N * (256 + 136)
    return {"workload": "decode attention, K and V q8_0-style (136 B per row), B16 Hq32 Hkv8 ctx 32768",
            "us_per_step": us, "n_splits": attn.params.n_splits, "algorithmic_bytes_per_step": algo,
            "achieved_gbs": algo / (us * 1e-6) / 1e9, "frac": algo / (us * 1e-6) / 1e9 / HBM_PEAK_GBS,
            "v_store": {"vectors": Hkv * N, "us_per_call": st_ms * 1e3, "gbs": st_bytes / (st_ms * 1e-3) / 1e9,
                        "note": "includes the allocation of the output buffer by the host wrapper"}}


def cache_maintenance_leg(torch, tqa, steps, warmup):
    """The kernels that rework a packed cache without the original vectors, on config 2's K tensor (262 144 vectors):
    temporal decay (tq_requantize 3 -> 2 bits), export to and import from the llama.cpp fork's per-vector blocks.
    Each is timed through the C ABI with the output allocated beforehand; bytes = the packed buffers read and written."""
    import ctypes
    from turboquant_plus_amd import _lib as L
    heads, tokens = 8, 32768
    c3, c2 = tqa.TurboCodec(3, seed=42), tqa.TurboCodec(2, seed=42)
    k = synth_kv(torch, heads, tokens, 900, outliers=4)
    packed3 = c3.store(k, kind="k")
    n3, n2 = tqa.packed_bytes(3, heads, tokens), tqa.packed_bytes(2, heads, tokens)
    fb = int(L.lib().tq_fork_block_bytes(3))
    out2 = torch.empty(n2, dtype=torch.uint8, device="cuda")
    blocks = torch.empty((heads, tokens, fb), dtype=torch.uint8, device="cuda")
    back3 = torch.empty(n3, dtype=torch.uint8, device="cuda")
    lib = L.lib()

    def requant(i):
        L.check(lib.tq_requantize(c3.handle.h, c2.handle.h, L.ptr(packed3), heads, tokens, L.KIND_K, L.ptr(out2), L.stream_ptr()))

    def export(i):
        L.check(lib.tq_export_fork_blocks(c3.handle.h, L.ptr(packed3), heads, tokens, L.KIND_K, L.ptr(blocks), L.stream_ptr()))

    def imp(i):
        L.check(lib.tq_import_fork_blocks(c3.handle.h, L.ptr(blocks), heads, tokens, L.KIND_K, L.ptr(back3), L.stream_ptr()))

    out = {"workload": "config 2's K tensor (8 heads x 32768 tokens, turbo3 codes) reworked in place of the original vectors"}
    for name, fn, nbytes in (("requantize_3to2", requant, n3 + n2), ("export_fork_blocks", export, n3 + heads * tokens * fb),
                             ("import_fork_blocks", imp, n3 + heads * tokens * fb)):
        _, ms = time_steps(torch, fn, steps, warmup)
        out[name] = {"us_per_call": ms * 1e3, "bytes": nbytes, "gbs": nbytes / (ms * 1e-3) / 1e9,
                     "frac": nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS}
    torch.cuda.synchronize()
    if not torch.equal(back3, packed3):
        raise RuntimeError("export followed by import changed the packed cache")
    # the same three on the V tensor: a token's codes are spread over the 64 rows of its tile, so these kernels stage a
    # block in LDS and work with sixteen lanes per token
    v = synth_kv(torch, heads, tokens, 901, outliers=0)
    packed3v = c3.store(v, kind="v")
    vt = {}
    for name, fn, nbytes in (
            ("requantize_3to2", lambda i: L.check(lib.tq_requantize(c3.handle.h, c2.handle.h, L.ptr(packed3v), heads, tokens, L.KIND_V, L.ptr(out2), L.stream_ptr())), n3 + n2),
            ("export_fork_blocks", lambda i: L.check(lib.tq_export_fork_blocks(c3.handle.h, L.ptr(packed3v), heads, tokens, L.KIND_V, L.ptr(blocks), L.stream_ptr())), n3 + heads * tokens * fb),
            ("import_fork_blocks", lambda i: L.check(lib.tq_import_fork_blocks(c3.handle.h, L.ptr(blocks), heads, tokens, L.KIND_V, L.ptr(back3), L.stream_ptr())), n3 + heads * tokens * fb)):
        _, ms = time_steps(torch, fn, steps, warmup)
        vt[name] = {"us_per_call": ms * 1e3, "frac": nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS}
    torch.cuda.synchronize()
    if not torch.equal(back3, packed3v):
        raise RuntimeError("export followed by import changed the packed V cache")
    out["v_tensor"] = vt
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=1000)
    ap.add_argument("--skip-cpu", action="store_true", help="omit the CPU baseline leg")
    ap.add_argument("--skip-small-batches", action="store_true",
                    help="decode leg without its small-batch shapes (counter runs: they launch the same kernel instantiation "
                         "as config 3, and a per-kernel mean would mix the shapes)")
    ap.add_argument("--legs", default="all",
                    help="comma-separated subset of store4,store3,decode,asym,tile,boundary,maintenance,peaks (profiling runs); "
                         "the JSON line then holds only those legs and is not the benchmark's line")
    ap.add_argument("--several-streams", action="store_true",
                    help="store legs: also time the launches issued round-robin on four streams (overlapping launches)")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also run a 1 GiB device copy (5x) so that FETCH_SIZE / WRITE_SIZE counters can be calibrated")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build measures one GPU; every (batch, kv-head) group and every vector is an "
              "independent unit, so more GPUs only replicate this number. Run with --gpus 1.", file=sys.stderr)
        sys.exit(2)
    import torch
    import turboquant_plus_amd as tqa
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the codec has no CPU path", file=sys.stderr)
        sys.exit(3)
    torch.cuda.set_device(0)
    # Bring the device out of idle before the first leg: a quarter of a second of plain device work, untimed and
    # apart from every leg's own W warm-up steps, so that the first leg does not start on a clock that is still
    # settling after the process's start-up (the store leg, which carries `value`, runs first).
    scratch = torch.zeros(1 << 26, dtype=torch.float32, device="cuda")
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < 0.25:
        for _ in range(20):
            scratch.add_(1.0)
        torch.cuda.synchronize()
    del scratch

    if args.copy_probe:
        src = torch.empty(1 << 28, dtype=torch.float32, device="cuda").normal_()
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    if args.legs != "all":
        legs = set(args.legs.split(","))
        part = {"partial_run": sorted(legs), "steps": args.steps, "warmup": args.warmup}
        if "store4" in legs:
            part["turbo4_store"] = store_leg(torch, tqa, 4, args.steps, args.warmup, several_streams=args.several_streams)
        if "store3" in legs:
            part["turbo3_store"] = store_leg(torch, tqa, 3, args.steps, args.warmup, several_streams=args.several_streams)
        if "decode" in legs:
            part["decode_attn"] = decode_leg(torch, tqa, args.steps, args.warmup, small_batches=not args.skip_small_batches)
        if "asym" in legs:
            part["asym_decode_q8k_turbo2v"] = asym_decode_leg(torch, tqa, max(10, args.steps // 4), max(2, args.warmup // 4))
        if "tile" in legs:
            part["score_tile"] = score_tile_leg(torch, tqa, args.steps, args.warmup)
        if "boundary" in legs:
            part["boundary_layer_q8k_q8v"] = boundary_layer_leg(torch, tqa, max(10, args.steps // 4), max(2, args.warmup // 4))
        if "maintenance" in legs:
            part["cache_maintenance"] = cache_maintenance_leg(torch, tqa, max(10, args.steps // 4), max(2, args.warmup // 4))
        if "peaks" in legs:
            part["measured_peaks"] = measured_peaks_leg(torch, tqa, args.steps, args.warmup)
        print(json.dumps(part, ensure_ascii=False))
        return
    s4 = store_leg(torch, tqa, 4, args.steps, args.warmup, several_streams=args.several_streams)
    s3 = store_leg(torch, tqa, 3, args.steps, args.warmup, several_streams=args.several_streams)
    dec = decode_leg(torch, tqa, args.steps, args.warmup, small_batches=not args.skip_small_batches)
    torch.cuda.empty_cache()
    asym = asym_decode_leg(torch, tqa, max(10, args.steps // 4), max(2, args.warmup // 4))
    torch.cuda.empty_cache()
    tile = score_tile_leg(torch, tqa, args.steps, args.warmup)
    torch.cuda.empty_cache()
    boundary = boundary_layer_leg(torch, tqa, max(10, args.steps // 4), max(2, args.warmup // 4))
    torch.cuda.empty_cache()
    maintenance = cache_maintenance_leg(torch, tqa, max(10, args.steps // 4), max(2, args.warmup // 4))
    torch.cuda.empty_cache()
    peaks = measured_peaks_leg(torch, tqa, args.steps, args.warmup)
    if args.skip_cpu:
        cpu_store = cpu_attn = None
    else:
        cpu_store, cpu_attn = cpu_baseline(4)
    dec["cpu_baseline"] = cpu_attn

    line = {
        # value: whole-job throughput over the K timed steps between two synchronisations (wall clock: it contains the gaps
        # between launches); roofline.achieved: the same bytes over the kernel's own duration (HIP events on the launch stream)
        "metric": METRIC, "value": s4["algorithmic_bytes_per_launch"] / (s4["ms_per_step"] * 1e-3) / 1e9, "unit": "GB/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": s4["ms_per_step"], "warmup_steps_run": s4["warmup_steps_run"],
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": s4["workload"], "global_batch": 2 * 8 * 32768, "io": "fp16 in, 4-bit codes + fp16 norm out",
                   "parallelism": "single GPU"},
        "roofline": {"bound": "hbm", "achieved": s4["gbs"], "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": s4["frac"],
                     "traffic": profile_traffic("store4")[0], "traffic_source": profile_traffic("store4")[1],
                     "kernel": "k_store_kv<4,4> (K and V of the layer, one launch per step)", "timed_blocks": s4["timed_blocks"],
                     "kernel_us": s4["kernel_us"],
                     "algorithmic_bytes_per_launch": s4["algorithmic_bytes_per_launch"]},
        "cpu_baseline": cpu_store,
        "turbo4_store": s4, "turbo3_store": s3, "decode_attn": dec, "asym_decode_q8k_turbo2v": asym,
        "score_tile": tile, "boundary_layer_q8k_q8v": boundary, "cache_maintenance": maintenance,
        "measured_peaks": peaks,
    }
    print(json.dumps(line, ensure_ascii=False))


if __name__ == "__main__":
    main()
