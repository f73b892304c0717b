#!/usr/bin/env python3
"""Benchmark of the block-quantized matmul path on one MI355X.

A step is one pass of the hot path over one prompt chunk: activation quantization (f32 -> int8 per 32) followed by the
Q4_K prefill GEMM of the benchmark definition's second configuration (weights 17408 x 5120 Q4_K, 8192 tokens).  Inputs are resident in HBM
when the timed region starts.  One JSON line is printed: the GEMM throughput in int8 TOP/s (2*M*N*K per step), the
roofline of the dominant kernel from per-launch HIP events, the decode GEMV bandwidth of config 3 as extra fields, and
the CPU baseline (the oracle's restatement of the reference's dequant + f32 matmul) timed on this host's cores.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_INT8_TOPS = 5000.0   # MI355X dense int8 MFMA, published
PEAK_HBM_GBS = 8000.0     # MI355X HBM3E, published
# HBM bytes one launch of the headline GEMM moves, from two counter runs of this script (FETCH_SIZE x 2.0 KiB read,
# WRITE_SIZE x 1.0 KiB written, the factors calibrated on the 2 GiB copy in the same runs): 1,338,862 KiB x 2 = 2742.0 MB
# read + 557,056 KiB = 570.4 MB written
GEMM_HBM_BYTES_PER_LAUNCH = 3.312e9


def log(*a):
    print(*a, file=sys.stderr, flush=True)


# After any idle period of more than a few milliseconds (host-side setup, a sleeping stream) this chip runs the first
# ~28 ms of a new burst of launches below the clock it then settles at: per-launch times of the headline GEMM go 2.74,
# 2.89, 2.74, 2.65, 2.59, 2.55, 2.49, 2.43, 2.38, 2.33, 2.30, then 2.29 ms for as long as the burst lasts; after a
# stream sync with no idle time behind it the next launch is at 2.29 again, after 5 ms idle at 2.43, after 20 ms the
# whole ramp repeats (one token's GEMV: 11.0 -> 10.64 us, two tokens' 14.8 -> 13.1 us).  Every timed region below
# therefore starts right behind SETTLE_MS of the same launches, untimed -- the sustained rate is what a prompt's or a
# generation's stream of matmuls sees -- and the headline reports how many steps that was ("settle_steps").
SETTLE_MS = 45.0


def settle(az, fn, cap=6000):
    """Runs fn() for about SETTLE_MS of device time (estimated from one launch), then syncs; returns the calls made.
    The estimate is taken from the second call: a sequence's first call also looks its kernels up in the code objects
    and touches its buffers for the first time (tens of ms for the expert layer), and an estimate that large cut the
    settling short, so that the timed region began inside the clock's ramp (the MoE layer read 0.78 instead of 0.71 ms
    whenever it was the first of its kind in the process)."""
    fn()
    az.Runtime.sync()
    e0 = az.Runtime.event()
    fn()
    e1 = az.Runtime.event()
    az.Runtime.sync()
    est = max(az.Runtime.elapsed_ms(e0, e1), 1e-3)
    az.Runtime.event_release(e0)
    az.Runtime.event_release(e1)
    n = int(min(cap, SETTLE_MS / est + 1))
    for _ in range(n):
        fn()
    az.Runtime.sync()
    return n + 2


def time_steps(az, fn, steps, warmup, after_warmup=None):
    settled = settle(az, fn)
    for _ in range(warmup):
        fn()
    az.Runtime.sync()
    if after_warmup is not None:
        after_warmup()
    e0 = az.Runtime.event()
    t0 = time.perf_counter()
    for _ in range(steps):
        fn()
    e1 = az.Runtime.event()
    az.Runtime.sync()
    wall = (time.perf_counter() - t0) * 1e3
    dev = az.Runtime.elapsed_ms(e0, e1)
    az.Runtime.event_release(e0)
    az.Runtime.event_release(e1)
    return dev / steps, wall / steps, settled


def bench_prefill(az, steps, warmup, M, N, K, qtype):
    eng = az.Engine(M, K)
    log(f"[bench] generating weights {N} x {K} and {M} x {K} activations ...")
    W = az.gen_weights(qtype, 1, N, K, 0.02)
    w = eng.make_weight(qtype, N, K, W)
    x = az.gen_normal(2, (M, K))
    xb = az.Runtime.from_numpy(x)
    cb = az.Runtime.alloc(M * N * 4)
    eng.profile(True)

    def step():
        eng.quantize(xb, K, K, M, M)
        eng.matmul("gemm", w, M, cb, N, 0, 0)

    def forget_warmup():   # the per-kernel statistics cover the timed launches only
        eng.profile_collect()
        eng.profile_reset()

    ms_dev, ms_wall, settled = time_steps(az, step, steps, warmup, forget_warmup)
    eng.profile_collect()
    gemm_ms, gemm_n = eng.profile_get("gemm")
    quant_ms, quant_n = eng.profile_get("quant_rows")
    gemm_min, gemm_med = eng.profile_stats("gemm")
    ops = 2.0 * M * N * K
    res = {
        "ms_per_step": ms_dev, "ms_per_step_wall": ms_wall, "tops": ops / (ms_dev * 1e-3) / 1e12,
        "gemm_kernel_ms": gemm_ms / max(gemm_n, 1), "quant_kernel_ms": quant_ms / max(quant_n, 1),
        "kernel_tops": ops / (gemm_ms / max(gemm_n, 1) * 1e-3) / 1e12, "ops": ops,
        "gemm_kernel_ms_min": gemm_min, "gemm_kernel_ms_median": gemm_med, "settle_steps": settled,
    }
    # parity spot check of what was just timed: sampled rows against the oracle
    try:
        import tests.oracle_lib as orc  # noqa: checker only
        y = cb.read(np.float32, M * N).reshape(M, N)
        aq, asc, _ = eng.read_activations(K, M)
        rows = np.arange(0, N, N // 64)[:64]
        toks = np.arange(0, M, M // 16)[:16]
        rb = az.gguf_bytes(qtype, 1, K)
        Wr = np.concatenate([W[r * rb:(r + 1) * rb] for r in rows])
        ref = orc.matmul_ref(qtype, Wr, len(rows), K, aq[toks], np.ascontiguousarray(asc[:, toks]))
        err = np.abs(y[np.ix_(toks, rows)] - ref).max(axis=1) / np.abs(ref).max(axis=1)
        res["parity_rel_err"] = float(err.max())
    except Exception as ex:  # the checker is optional for the measurement
        res["parity_rel_err"] = None
        log(f"[bench] parity spot check skipped: {ex}")
    for b in (cb, xb):
        b.free()
    w.free()
    eng.close()
    return res, W


def bench_decode(az, qtype, N, K, T, launches, copies):
    """GEMV over `copies` distinct weight buffers in turn (more bytes than the 256 MB last-level cache holds)."""
    eng = az.Engine(16, K)
    W = az.gen_weights(qtype, 3, N, K, 0.02)
    ws = [eng.make_weight(qtype, N, K, W) for _ in range(copies)]
    x = az.gen_normal(4, (T, K))
    xb = az.Runtime.from_numpy(x)
    eng.quantize(xb, K, K, 16, T)
    cb = az.Runtime.alloc((T if T <= 8 else 16) * N * 4)   # (9-16 tokens: a chunk of 16 rows)
    def round_of_copies():   # warm-up: every buffer in turn
        for i in range(copies):
            eng.matmul("gemv", ws[i], 16, cb, N, 0, 0)
    settle(az, round_of_copies)
    # (a) launches back to back between two events on the stream: launch-to-launch time, no per-launch event pair
    e0 = az.Runtime.event()
    for i in range(launches):
        eng.matmul("gemv", ws[i % copies], 16, cb, N, 0, 0)
    e1 = az.Runtime.event()
    az.Runtime.sync()
    batch_us = az.Runtime.elapsed_ms(e0, e1) / launches * 1e3
    az.Runtime.event_release(e0)
    az.Runtime.event_release(e1)
    # (b) an event pair around every launch (adds the events' own latency to a kernel of a few microseconds)
    eng.profile(True)
    for i in range(launches):
        eng.matmul("gemv", ws[i % copies], 16, cb, N, 0, 0)
    eng.profile_collect()
    ms, n = eng.profile_get("gemv")
    bytes_alg = az.gguf_bytes(qtype, N, K) + T * (K + K // 32 * 4 + K // 16 * 2) + T * N * 4
    gbs = bytes_alg / (batch_us * 1e-6) / 1e9
    for wt in ws:
        wt.free()
    cb.free()
    xb.free()
    eng.close()
    return {"kernel_us": batch_us, "per_launch_event_us": ms / n * 1e3, "bytes": bytes_alg, "GBps": gbs,
            "frac_hbm_peak": gbs / PEAK_HBM_GBS, "launches": n,
            "distinct_weight_MB": copies * az.gguf_bytes(qtype, N, K) / 1e6}


def bench_launch_list(az, N=2048, layers=32, reps=40):
    """A decode-like chain of small launches -- `layers` times (quantize one token, GEMV N x N Q4_K) -- issued launch
    by launch and as one recorded list (arcz_record_begin / arcz_list_run): device time per launch, both ways."""
    eng = az.Engine(16, N)
    W = az.gen_weights(az.Q4_K, 9, N, N, 0.02)
    ws = [eng.make_weight(az.Q4_K, N, N, W) for _ in range(4)]
    bufs = [az.Runtime.from_numpy(az.gen_normal(10, (1, N))), az.Runtime.alloc(N * 4)]

    def step():
        for i in range(layers):
            eng.quantize(bufs[i % 2], N, N, 16, 1)
            eng.matmul("chain", ws[i % 4], 16, bufs[(i + 1) % 2], N, 0, 0)

    def timed(fn):
        settle(az, fn)
        e0 = az.Runtime.event()
        for _ in range(reps):
            fn()
        e1 = az.Runtime.event()
        az.Runtime.sync()
        ms = az.Runtime.elapsed_ms(e0, e1)
        az.Runtime.event_release(e0)
        az.Runtime.event_release(e1)
        return ms

    step()
    lst = az.Runtime.record(step)
    n = lst.launches
    eager_ms, list_ms = timed(step), timed(lst.run)
    lst.free()
    for w in ws:
        w.free()
    for b in bufs:
        b.free()
    eng.close()
    return {"launches_per_step": int(n), "eager_us_per_launch": eager_ms / reps / n * 1e3,
            "list_us_per_launch": list_ms / reps / n * 1e3, "eager_us_per_step": eager_ms / reps * 1e3,
            "list_us_per_step": list_ms / reps * 1e3, "shape": [N, N], "layers": layers}


def bench_types(az, N=17408, K=5120):
    """Every weight type on the headline matrix: GEMV over 1, 2, 8 and 16 tokens (cycling through distinct weight
    buffers, as bench_decode) and the prefill GEMM at 2048 tokens.  Not part of the default run (--types)."""
    names = {az.Q4_0: "Q4_0", az.Q8_0: "Q8_0", az.Q3_K: "Q3_K", az.Q4_K: "Q4_K", az.Q5_K: "Q5_K", az.Q6_K: "Q6_K",
             az.IQ3_XXS: "IQ3_XXS", az.IQ4_NL: "IQ4_NL", az.IQ3_S: "IQ3_S", az.IQ4_XS: "IQ4_XS", az.MXFP4: "MXFP4"}
    out = {}
    for qt, name in names.items():
        copies = 6
        row = {"gguf_MB": az.gguf_bytes(qt, N, K) / 1e6, "device_MB": az.planes_bytes(qt, N, K) / 1e6}
        for T in (1, 2, 8, 16):
            d = bench_decode(az, qt, N, K, T, 200, copies)
            row[f"T{T}_us"] = d["kernel_us"]
            row[f"T{T}_frac_hbm_peak"] = d["frac_hbm_peak"]
        r, _ = bench_gemm_config(az, qt, N, K, 2048, 5, 61)
        row["M2048_ms"], row["M2048_TOPS"] = r["ms"], r["TOPS"]
        out[name] = row
        log(f"[bench] {name} {N}x{K}: {row}")
    return out


def bench_gemv_gu(az, qtype, F, K, launches, copies):
    """Gate and up of one token in one launch (Engine::gemv_gu), over `copies` distinct pairs of matrices in turn."""
    eng = az.Engine(16, K)
    Wg, Wu = az.gen_weights(qtype, 5, F, K, 0.02), az.gen_weights(qtype, 6, F, K, 0.02)
    ws = [(eng.make_weight(qtype, F, K, Wg), eng.make_weight(qtype, F, K, Wu)) for _ in range(copies)]
    xb = az.Runtime.from_numpy(az.gen_normal(4, (1, K)))
    eng.quantize(xb, K, K, 16, 1)
    cb = az.Runtime.alloc(2 * F * 4)
    def round_of_copies():
        for g, u in ws:
            assert eng.gemv_gu(g, u, 16, cb)
    settle(az, round_of_copies)
    e0 = az.Runtime.event()
    for i in range(launches):
        eng.gemv_gu(ws[i % copies][0], ws[i % copies][1], 16, cb)
    e1 = az.Runtime.event()
    az.Runtime.sync()
    us = az.Runtime.elapsed_ms(e0, e1) / launches * 1e3
    az.Runtime.event_release(e0)
    az.Runtime.event_release(e1)
    nbytes = 2 * az.gguf_bytes(qtype, F, K) + (K + K // 32 * 4 + K // 16 * 2) + 2 * F * 4
    for g, u in ws:
        g.free()
        u.free()
    cb.free()
    xb.free()
    eng.close()
    return {"kernel_us": us, "bytes": nbytes, "GBps": nbytes / us / 1e3, "frac_hbm_peak": nbytes / us / 1e3 / PEAK_HBM_GBS,
            "launches": launches, "distinct_weight_MB": 2 * copies * az.gguf_bytes(qtype, F, K) / 1e6}


def bench_gemm_config(az, qtype, N, K, M, launches, seed, W=None):
    """One GEMM (or GEMV-form, M <= 8) configuration: per-launch device time from events around `launches` launches."""
    eng = az.Engine(max(M, 16), K)
    if W is None:
        W = az.gen_weights(qtype, seed, N, K, 0.02)
    w = eng.make_weight(qtype, N, K, W)
    Mp = M if M > 8 else 16
    xb = az.Runtime.from_numpy(az.gen_normal(seed + 1, (M, K)))
    eng.quantize(xb, K, K, Mp, M)
    cb = az.Runtime.alloc(max(M, 1) * N * 4)
    settle(az, lambda: eng.matmul("cfg", w, Mp, cb, N, 0, 0))
    e0 = az.Runtime.event()
    for _ in range(launches):
        eng.matmul("cfg", w, Mp, cb, N, 0, 0)
    e1 = az.Runtime.event()
    az.Runtime.sync()
    ms = az.Runtime.elapsed_ms(e0, e1) / launches
    az.Runtime.event_release(e0)
    az.Runtime.event_release(e1)
    ops = 2.0 * M * N * K
    nbytes = az.gguf_bytes(qtype, N, K) + M * (K + K // 32 * 4 + K // 16 * 2) + M * N * 4
    for b in (cb, xb):
        b.free()
    w.free()
    eng.close()
    return {"M": M, "N": N, "K": K, "ms": ms, "TOPS": ops / (ms * 1e-3) / 1e12,
            "frac_int8_peak": ops / (ms * 1e-3) / 1e12 / PEAK_INT8_TOPS, "GBps": nbytes / (ms * 1e-3) / 1e9,
            "frac_hbm_peak": nbytes / (ms * 1e-3) / 1e9 / PEAK_HBM_GBS}, W


def bench_moe(az, launches, ready_made=True):
    """The MoE configuration (configs[4] of the benchmark definition): 128 experts, top-8, 4096 tokens, hidden 2048, expert FFN 768, Q4_K; the whole layer
    (route, sort, gate/up tile GEMM with SwiGLU, expert-input quantization, down tile GEMM, combine) per launch.
    ready_made=False: an engine made with ARCZ_MOE_PRE=0 (the tile kernels form their scale vectors per tile and step
    instead of taking them ready-made from 8 more bytes per 32 expert weights)."""
    NE, NU, T, E, F, qt = 128, 8, 4096, 2048, 768, az.Q4_K
    before = os.environ.get("ARCZ_MOE_PRE")
    os.environ["ARCZ_MOE_PRE"] = "1" if ready_made else "0"
    try:
        eng = az.Engine(T, E)   # (reads the switch here)
    finally:
        if before is None:
            del os.environ["ARCZ_MOE_PRE"]
        else:
            os.environ["ARCZ_MOE_PRE"] = before
    Wg = az.gen_weights(qt, 21, NE * F, E, 0.02)
    Wu = az.gen_weights(qt, 22, NE * F, E, 0.02)
    Wd = az.gen_weights(qt, 23, NE * E, F, 0.02)
    L = eng.make_moe_layer(qt, Wg, Wu, Wd, NE, NU, E, F)
    del Wg, Wu, Wd
    xb = az.Runtime.from_numpy(az.gen_normal(24, (T, E)))
    lb = az.Runtime.from_numpy(az.gen_normal(25, (T, NE)))
    ob = az.Runtime.alloc(T * E * 4).fill(0)
    eng.quantize(xb, E, E, T, T)
    settle(az, lambda: eng.layer_moe(L, lb, NE, ob, T, T))
    # the layer's time: launches back to back between two events, no event pair around each kernel (a pair costs 2.5-3 us,
    # and the layer is six kernels) ...
    e0 = az.Runtime.event()
    for _ in range(launches):
        eng.layer_moe(L, lb, NE, ob, T, T)
    e1 = az.Runtime.event()
    az.Runtime.sync()
    ms = az.Runtime.elapsed_ms(e0, e1) / launches
    az.Runtime.event_release(e0)
    az.Runtime.event_release(e1)
    # ... and, right behind them, the same launches again with the per-kernel events, for the parts
    eng.profile(True)
    for _ in range(launches):
        eng.layer_moe(L, lb, NE, ob, T, T)
    az.Runtime.sync()
    eng.profile_collect()
    parts = {}
    for name in ("moe_route", "moe_scan", "moe_scatter", "moe_gateup", "moe_quant", "moe_down", "moe_combine"):
        t, n = eng.profile_get(name)
        parts[name + "_ms"] = t / launches   # per layer, however many launches the step takes
    ops = T * NU * 3 * 2.0 * F * E
    gemm_ms = parts["moe_gateup_ms"] + parts["moe_down_ms"]
    for b in (xb, lb, ob):
        b.free()
    eng.close()
    return {"tokens": T, "experts": NE, "top": NU, "hidden": E, "ffn": F, "layer_ms": ms, "ops": ops,
            "layer_TOPS": ops / (ms * 1e-3) / 1e12, "gemm_kernels_ms": gemm_ms,
            "gemm_TOPS": ops / (gemm_ms * 1e-3) / 1e12, "gemm_frac_int8_peak": ops / (gemm_ms * 1e-3) / 1e12 / PEAK_INT8_TOPS,
            **parts}


def bench_moe_decode(az, launches):
    """The same layer for passes of 1 to 16 tokens (the matrix-vector expert kernels): microseconds per layer,
    launches back to back."""
    NE, NU, E, F, qt = 128, 8, 2048, 768, az.Q4_K
    eng = az.Engine(16, E)
    L = eng.make_moe_layer(qt, az.gen_weights(qt, 21, NE * F, E, 0.02), az.gen_weights(qt, 22, NE * F, E, 0.02),
                           az.gen_weights(qt, 23, NE * E, F, 0.02), NE, NU, E, F)
    out = {}
    for T in (1, 2, 4, 8, 16):
        xb = az.Runtime.from_numpy(az.gen_normal(24, (T, E)))
        lb = az.Runtime.from_numpy(az.gen_normal(25 + T, (T, NE)))
        ob = az.Runtime.alloc(T * E * 4).fill(0)
        eng.quantize(xb, E, E, 16, T)
        settle(az, lambda: eng.layer_moe(L, lb, NE, ob, T, 16))
        e0 = az.Runtime.event()
        for _ in range(launches):
            eng.layer_moe(L, lb, NE, ob, T, 16)
        e1 = az.Runtime.event()
        az.Runtime.sync()
        out[f"T{T}_layer_us"] = az.Runtime.elapsed_ms(e0, e1) / launches * 1e3
        az.Runtime.event_release(e0)
        az.Runtime.event_release(e1)
        for b in (xb, lb, ob):
            b.free()
    eng.close()
    return out


def bench_producers(az, M, K, copies=4):
    """The fused producers at the headline chunk's shape: RMS norm + quantization of M rows of K, SwiGLU + quantization
    of M rows of [gate(K) | up(K)]; HBM bytes = f32 rows read once + int8 rows, scales and sums written.  The launches
    go round `copies` distinct inputs (4 x 168 MB, 4 x 336 MB for SwiGLU: more than the 256 MB last-level cache holds),
    so the rates are HBM rates."""
    eng = az.Engine(M, K)
    xs = [az.Runtime.from_numpy(az.gen_normal(51 + i, (M, K))) for i in range(copies)]
    wb = az.Runtime.from_numpy(np.ones(K, np.float32))
    g0 = az.gen_normal(52, (M, 2 * K))
    gs = [az.Runtime.from_numpy(g0) for _ in range(copies)]
    del g0
    out = {}
    for name, fn, rd in (("rmsnorm_quant", lambda i: eng.rmsnorm_quant(xs[i], 0, wb, K, M, M, 1e-6), 4.0 * M * K),
                         ("swiglu_quant", lambda i: eng.swiglu_quant(gs[i], K, M, M), 8.0 * M * K),
                         ("quant_rows", lambda i: eng.quantize(xs[i], K, K, M, M), 4.0 * M * K)):
        def round_of_copies():
            for i in range(copies):
                fn(i)
        settle(az, round_of_copies)
        e0 = az.Runtime.event()
        for it in range(20):
            fn(it % copies)
        e1 = az.Runtime.event()
        az.Runtime.sync()
        us = az.Runtime.elapsed_ms(e0, e1) / 20 * 1e3
        az.Runtime.event_release(e0)
        az.Runtime.event_release(e1)
        nbytes = rd + M * K * (1 + 4 / 32 + 2 / 16)
        out[name] = {"us": us, "GBps": nbytes / us / 1e3, "frac_hbm_peak": nbytes / us / 1e3 / PEAK_HBM_GBS}
    out["shape"] = [M, K]
    out["note"] = f"back-to-back launches cycling through {copies} distinct inputs (more than the last-level cache holds)"
    for b in xs + gs + [wb]:
        b.free()
    eng.close()
    return out


def bench_probes(az):
    """What the machine itself delivers: a streaming read and a copy over 2 GiB, and the issue rate of register-resident
    int8 matrix instructions."""
    n = 2 << 30
    src = az.Runtime.alloc(n).fill(0x01020304)
    dst = az.Runtime.alloc(n)
    sink = az.Runtime.alloc(64).fill(0)
    cus = az.Runtime.cus()
    out = {}
    k = az.Runtime.kernel("ops", "", "read_probe")
    grid = (cus * 8 * 256,)
    best = 1e9
    for _ in range(5):
        best = min(best, az.Runtime.launch(k, grid, (256,), [src, ("z", n // 16), sink], timed=True))
    out["read_GBps"] = n / (best * 1e-3) / 1e9
    k = az.Runtime.kernel("ops", "", "copy128")
    best = 1e9
    for _ in range(5):
        best = min(best, az.Runtime.launch(k, grid, (256,), [src, dst, ("z", n // 16)], timed=True))
    out["copy_GBps_read_plus_write"] = 2 * n / (best * 1e-3) / 1e9
    k = az.Runtime.kernel("ops", "", "mfma_probe")
    iters, wgs = 20000, cus * 8
    best = 1e9
    for _ in range(3):
        best = min(best, az.Runtime.launch(k, (wgs * 256,), (256,), [sink, iters], timed=True))
    out["int8_mfma_issue_TOPS"] = 2.0 * 32 * 32 * 32 * 4 * iters * wgs * 4 / (best * 1e-3) / 1e12
    for b in (src, dst, sink):
        b.free()
    return out


def cpu_baseline(az, W, qtype, N, K, budget_s=15.0):
    """The oracle's restatement of the reference CPU matmul (dequant row -> double-accumulated dots, OpenMP over rows;
    tools/ref_forward.cpp:251-305), all host cores, on a bounded sample of config 2 (the first rows x tokens that fit
    the time budget), and on config 1 (Q8_0 4096 x 4096, 512 tokens) in full."""
    import tests.oracle_lib as orc
    rb = az.gguf_bytes(qtype, 1, K)
    M = 8192
    xc = az.gen_normal(2, (256, K))
    aqc, ascc, _ = orc.quantize_act(xc)
    orc.matmul_ref(qtype, W[:64 * rb], 64, K, aqc, ascc)          # warm the threads up
    t0 = time.perf_counter()
    orc.matmul_ref(qtype, W[:1024 * rb], 1024, K, aqc, ascc)      # calibration
    rate = 2.0 * 256 * 1024 * K / max(time.perf_counter() - t0, 1e-3)
    # all weight rows, and as many of the 8192 tokens as the budget allows (in steps of 256); fewer rows on a slow host
    toks = int(min(M, max(256, budget_s * rate / (2.0 * N * K) // 256 * 256)))
    rows = N if toks > 256 else int(min(N, max(512, budget_s * rate / (2.0 * 256 * K) // 16 * 16)))
    x = az.gen_normal(2, (M, K))[:toks]
    aq, asc, _ = orc.quantize_act(np.ascontiguousarray(x))
    t0 = time.perf_counter()
    orc.matmul_ref(qtype, W[:rows * rb], rows, K, aq, asc)
    dt = time.perf_counter() - t0
    ops = 2.0 * toks * rows * K
    # config 1 in full
    N1, K1, M1 = 4096, 4096, 512
    W1 = az.gen_weights(az.Q8_0, 31, N1, K1, 0.02)
    aq1, asc1, _ = orc.quantize_act(az.gen_normal(32, (M1, K1)))
    t0 = time.perf_counter()
    orc.matmul_ref(az.Q8_0, W1, N1, K1, aq1, asc1)
    dt1 = time.perf_counter() - t0
    return {"value": ops / dt / 1e12, "unit": "TOP/s", "cores": orc.num_threads(), "kind": "port",
            "sample": f"first {rows} of {N} weight rows x first {toks} of {M} tokens, K={K}: {dt:.2f} s "
                      f"({ops / dt / 1e9:.1f} G op/s of 2*M*N*K; dequant row + double-accumulated dot, OpenMP)",
            "config1_full": {"workload": "Q8_0 4096x4096, 512 tokens", "seconds": dt1,
                             "TOPS": 2.0 * M1 * N1 * K1 / dt1 / 1e12}}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-decode", action="store_true", help="skip the decode GEMV extras")
    ap.add_argument("--types", action="store_true",
                    help="only the table of all weight types on the headline matrix (one JSON line, key weight_types)")
    ap.add_argument("--no-extras", action="store_true",
                    help="skip the other configurations (Q8_0 GEMM, Q6_K output head, MoE layer) and the machine probes")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU only (no collectives, no sharding); use --gpus 1")

    import arcinferzero_amd as az
    az.Runtime.init(0)
    log(f"[bench] {az.Runtime.device_name()}, {az.Runtime.cus()} CUs")
    if args.types:
        print(json.dumps({"weight_types": bench_types(az)}))
        return
    M, N, K, qtype = 8192, 17408, 5120, az.Q4_K
    pre, W = bench_prefill(az, args.steps, args.warmup, M, N, K, qtype)
    log(f"[bench] prefill: {pre}")
    out = {
        "metric": "prefill int8-GEMM TOPS & %MFMA peak; decode GEMV GB/s & %HBM peak",
        "value": pre["tops"], "unit": "TOP/s (2*M*N*K int8 ops per step)", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "settle_steps": pre["settle_steps"], "ms_per_step": pre["ms_per_step"], "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "int8 x int8 -> int32 block sums, f32 scale application", "data": "synthetic",
        "config": {"workload": "Q4_K dense prefill GEMM: weights 17408x5120 Q4_K, activations 8192x5120 f32 "
                               "quantized to int8 per 32 in the step, out 8192x17408 f32 (configs[1] of the benchmark definition)",
                   "M": M, "N": N, "K": K, "step": "quant_rows + gemm"},
        "roofline": {"bound": "mfma", "achieved": pre["kernel_tops"], "peak": PEAK_INT8_TOPS, "unit": "TOP/s",
                     "frac": pre["kernel_tops"] / PEAK_INT8_TOPS,
                     # what the vector unit allows whatever the matrix unit does: per 32 x 32 x 32 int8 product (32
                     # cycles of the matrix unit at the published peak) a lane converts 16 int32 sums and multiplies
                     # them into 16 f32 accumulators with the block's scale tile: 32 vector instructions x 4 cycles
                     "ceiling_frac": 0.25,
                     "ceiling": "per-32 scales: 2 vector instructions (int32 -> f32, fma with the scale tile) per "
                                "accumulator and block = 128 vector cycles per 32-cycle matrix instruction",
                     "traffic": GEMM_HBM_BYTES_PER_LAUNCH,
                     "traffic_source": "profiles/bench_hbm_traffic_fetch_write.txt (counter runs of this script; "
                                       "a constant here, not read in this run)",
                     "kernel": "gemm__QTYPE12_ACT321_AU3",
                     "kernel_ms": pre["gemm_kernel_ms"], "kernel_ms_median": pre["gemm_kernel_ms_median"],
                     "kernel_ms_min": pre["gemm_kernel_ms_min"], "ops_per_launch": pre["ops"]},
        "parity_rel_err_sampled": pre["parity_rel_err"],
        "quant_kernel_ms": pre["quant_kernel_ms"],
    }
    if not args.no_decode:
        d1 = bench_decode(az, az.Q4_K, 17408, 5120, 1, 200, 8)
        log(f"[bench] decode T=1: {d1}")
        d2 = bench_decode(az, az.Q4_K, 5120, 17408, 2, 200, 8)
        log(f"[bench] decode T=2: {d2}")
        dgu = bench_gemv_gu(az, az.Q4_K, 17408, 5120, 200, 4)
        log(f"[bench] decode gate + up in one launch: {dgu}")
        # a batch of 8 tokens (the matrix-pipe GEMV): the headline matrix, and the Q6_K down projection's shape
        d8 = bench_decode(az, az.Q4_K, 17408, 5120, 8, 200, 8)
        log(f"[bench] decode T=8: {d8}")
        d86 = bench_decode(az, az.Q6_K, 5120, 17408, 8, 200, 6)
        log(f"[bench] decode T=8 Q6_K: {d86}")
        dll = bench_launch_list(az)
        log(f"[bench] chain of small launches, eager and as a recorded list: {dll}")
        out["decode"] = {"launch_list_chain_Q4_K_2048x2048_T1": dll, "Q4_K_17408x5120_T1": d1, "Q4_K_5120x17408_T2": d2, "Q4_K_gate_up_2x17408x5120_T1": dgu,
                         "Q4_K_17408x5120_T8": d8, "Q6_K_5120x17408_T8": d86, "hbm_peak_GBps": PEAK_HBM_GBS}
    if not args.no_extras:
        az.self_check()
        c1, _ = bench_gemm_config(az, az.Q8_0, 4096, 4096, 512, 50, 31)
        log(f"[bench] Q8_0 4096x4096 M=512: {c1}")
        out["other_configs"] = {"Q8_0_4096x4096_M512": c1}
        W6 = None
        for M6, launches in ((1, 50), (64, 20), (2048, 3)):
            r, W6 = bench_gemm_config(az, az.Q6_K, 151936, 5120, M6, launches, 41, W6)
            log(f"[bench] Q6_K 151936x5120 M={M6}: {r}")
            out["other_configs"][f"Q6_K_151936x5120_M{M6}"] = r
        del W6
        # Q5_K (one of the further weight types): the same matrix as the headline, one token and 8192
        out["other_configs"]["Q5_K_17408x5120_T1"] = bench_decode(az, az.Q5_K, 17408, 5120, 1, 200, 8)
        r5, _ = bench_gemm_config(az, az.Q5_K, 17408, 5120, 8192, 3, 51)
        out["other_configs"]["Q5_K_17408x5120_M8192"] = r5
        log(f"[bench] Q5_K 17408x5120: {out['other_configs']['Q5_K_17408x5120_T1']} {r5}")
        out["other_configs"]["MoE_128x8_T4096_E2048_F768_Q4_K"] = bench_moe(az, 5)
        log(f"[bench] MoE: {out['other_configs']['MoE_128x8_T4096_E2048_F768_Q4_K']}")
        out["other_configs"]["MoE_128x8_T4096_E2048_F768_Q4_K_scales_in_kernel"] = bench_moe(az, 5, ready_made=False)
        log(f"[bench] MoE, ARCZ_MOE_PRE=0: {out['other_configs']['MoE_128x8_T4096_E2048_F768_Q4_K_scales_in_kernel']}")
        out["other_configs"]["MoE_128x8_E2048_F768_Q4_K_decode"] = bench_moe_decode(az, 50)
        log(f"[bench] MoE decode: {out['other_configs']['MoE_128x8_E2048_F768_Q4_K_decode']}")
        out["producers_8192x5120"] = bench_producers(az, M, K)
        log(f"[bench] producers: {out['producers_8192x5120']}")
        out["machine_probes"] = bench_probes(az)
        log(f"[bench] probes: {out['machine_probes']}")
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(az, W, qtype, N, K)
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
