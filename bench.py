#!/usr/bin/env python3
"""Benchmark of the block-quantized matmul path on one MI355X.

A step is one pass of the hot path over one prompt chunk: activation quantization (f32 -> int8 per 32) followed by the
Q4_K prefill GEMM of BASELINE.json's config 2 (weights 17408 x 5120 Q4_K, 8192 tokens).  Inputs are resident in HBM
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


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def time_steps(az, fn, steps, warmup):
    for _ in range(warmup):
        fn()
    az.Runtime.sync()
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
    return dev / steps, wall / steps


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

    ms_dev, ms_wall = time_steps(az, step, steps, warmup)
    eng.profile_collect()
    gemm_ms, gemm_n = eng.profile_get("gemm")
    quant_ms, quant_n = eng.profile_get("quant_rows")
    ops = 2.0 * M * N * K
    res = {
        "ms_per_step": ms_dev, "ms_per_step_wall": ms_wall, "tops": ops / (ms_dev * 1e-3) / 1e12,
        "gemm_kernel_ms": gemm_ms / max(gemm_n, 1), "quant_kernel_ms": quant_ms / max(quant_n, 1),
        "kernel_tops": ops / (gemm_ms / max(gemm_n, 1) * 1e-3) / 1e12, "ops": ops,
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
    cb = az.Runtime.alloc(T * N * 4)
    for i in range(copies):   # warm-up: every buffer once
        eng.matmul("gemv", ws[i], 16, cb, N, 0, 0)
    az.Runtime.sync()
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


def cpu_baseline(az, W, qtype, N, K, budget_s=12.0):
    """The oracle's restatement of the reference CPU matmul (dequant row -> double-accumulated dots), all host cores,
    on a bounded sample of config 2: the first rows x tokens that fit the time budget."""
    import tests.oracle_lib as orc
    rb = az.gguf_bytes(qtype, 1, K)
    x = az.gen_normal(2, (64, K))
    aq, asc, _ = orc.quantize_act(x)
    t0 = time.perf_counter()
    orc.matmul_ref(qtype, W[:256 * rb], 256, K, aq, asc)
    dt = time.perf_counter() - t0
    rate = 2.0 * 64 * 256 * K / max(dt, 1e-6)
    toks = 256
    rows = int(min(N, max(256, budget_s * rate / (2.0 * toks * K))))
    rows -= rows % 16
    x = az.gen_normal(2, (toks, K))
    aq, asc, _ = orc.quantize_act(x)
    t0 = time.perf_counter()
    orc.matmul_ref(qtype, W[:rows * rb], rows, K, aq, asc)
    dt = time.perf_counter() - t0
    ops = 2.0 * toks * rows * K
    return {"value": ops / dt / 1e12, "unit": "TOP/s", "cores": orc.num_threads(), "kind": "port",
            "sample": f"first {rows} of {N} weight rows x first {toks} of 8192 tokens, K={K}: {dt:.2f} s "
                      f"({ops / dt / 1e9:.1f} GFLOP/s of 2*M*N*K; dequant row + double-accumulated dot, OpenMP)"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-decode", action="store_true", help="skip the decode GEMV extras")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU only (no collectives, no sharding); use --gpus 1")

    import arcinferzero_amd as az
    az.Runtime.init(0)
    log(f"[bench] {az.Runtime.device_name()}, {az.Runtime.cus()} CUs")
    M, N, K, qtype = 8192, 17408, 5120, az.Q4_K
    pre, W = bench_prefill(az, args.steps, args.warmup, M, N, K, qtype)
    log(f"[bench] prefill: {pre}")
    out = {
        "metric": "prefill int8-GEMM TOPS & %MFMA peak; decode GEMV GB/s & %HBM peak",
        "value": pre["tops"], "unit": "TOP/s (2*M*N*K int8 ops per step)", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": pre["ms_per_step"], "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "int8 x int8 -> int32 block sums, f32 scale application", "data": "synthetic",
        "config": {"workload": "Q4_K dense prefill GEMM: weights 17408x5120 Q4_K, activations 8192x5120 f32 "
                               "quantized to int8 per 32 in the step, out 8192x17408 f32 (BASELINE configs[1])",
                   "M": M, "N": N, "K": K, "step": "quant_rows + gemm"},
        "roofline": {"bound": "mfma", "achieved": pre["kernel_tops"], "peak": PEAK_INT8_TOPS, "unit": "TOP/s",
                     "frac": pre["kernel_tops"] / PEAK_INT8_TOPS, "traffic": None, "kernel": "gemm__QTYPE12_ACT321",
                     "kernel_ms": pre["gemm_kernel_ms"], "ops_per_launch": pre["ops"]},
        "parity_rel_err_sampled": pre["parity_rel_err"],
        "quant_kernel_ms": pre["quant_kernel_ms"],
    }
    if not args.no_decode:
        d1 = bench_decode(az, az.Q4_K, 17408, 5120, 1, 200, 8)
        log(f"[bench] decode T=1: {d1}")
        d2 = bench_decode(az, az.Q4_K, 5120, 17408, 2, 200, 8)
        log(f"[bench] decode T=2: {d2}")
        out["decode"] = {"Q4_K_17408x5120_T1": d1, "Q4_K_5120x17408_T2": d2, "hbm_peak_GBps": PEAK_HBM_GBS}
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(az, W, qtype, N, K)
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
