#!/usr/bin/env python3
"""Benchmark of the Q4_0 hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

One step = one pass over the LLaMA-7B-shaped Q4_0 decode GEMV set at batch 1 (BASELINE.json
configs[1]): K=4096->N=4096, K=4096->N=11008, K=11008->N=4096, K=4096->N=32000, f32
activations N(0,1), weights N(0,0.02) quantized to Q4_0 on the device.  Successive steps
rotate over distinct copies of the weights totalling more than 1 GB so that every launch
streams from HBM rather than from the 256 MB Infinity Cache.  Inputs are resident in HBM
before the timed region; timing is by HIP events on the stream the kernels run on.

Prints ONE JSON line.  `value` is weight bytes per second over the whole step (GB/s);
`roofline` prices the GEMV kernel against the 8 TB/s HBM peak; `cpu_baseline` is the
reference's CPU algorithm (Q8_0 activations + integer dot, 4 worker threads as the
reference hard-codes) timed on this host on a bounded sample of the same workload.
The prefill matmul (configs[2]) and the row kernels (configs[3]) are reported under
`extra`, each against its own roofline.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0          # MI355X HBM3E, published
MFMA_F16_PEAK_TFLOPS = 2500.0   # MI355X dense fp16 MFMA, published
GEMV_SHAPES = [(4096, 4096), (4096, 11008), (11008, 4096), (4096, 32000)]  # (K, N)
PREFILL = (512, 4096, 11008)    # (M, K, N)
ROTATE_BYTES = 1200 << 20
# HBM bytes per GEMV launch (average over the four shapes) measured with rocprofv3 --pmc FETCH_SIZE and
# WRITE_SIZE on this workload, each scaled by what the same counter reads for a device-to-device copy of
# known size (FETCH_SIZE x 2.000, WRITE_SIZE x 1.000); see profiles/gemv_q4_0_dot8__llama7b_gemv_set.md
GEMV_TRAFFIC_BYTES_PER_LAUNCH = 33779200


def q4_bytes(k, n):
    return n * (k // 32) * 18


def make_q4_matrix(dev, rng, k, n):
    """Weights N(0, 0.02) drawn on the host in slabs, quantized to Q4_0 on the device."""
    out = dev.alloc(q4_bytes(k, n))
    rows_per_slab = max(1, (64 << 20) // (4 * k))
    stage = dev.alloc(rows_per_slab * k * 4)
    for r0 in range(0, n, rows_per_slab):
        r1 = min(n, r0 + rows_per_slab)
        w = rng.standard_normal((r1 - r0, k), dtype=np.float32) * np.float32(0.02)
        dev.upload(w, stage)
        dev.quantize_row_q4_0(stage, out.view(q4_bytes(k, r0)), (r1 - r0) * k)
    dev.synchronize()
    dev.free(stage)
    return out


def timed(dev, fn, iters, reps=1):
    """Median over `reps` of the event-timed duration (ms) of `iters` calls of fn(i)."""
    e0, e1 = dev.event(), dev.event()
    out = []
    for _ in range(reps):
        dev.synchronize()
        dev.record(e0)
        for i in range(iters):
            fn(i)
        dev.record(e1)
        out.append(dev.elapsed_ms(e0, e1))
        dev.synchronize()
    dev.event_destroy(e0)
    dev.event_destroy(e1)
    return float(np.median(out))


def cpu_baseline(weights_host, xs_host, budget_s):
    """The reference CPU op restated in C (oracle/), timed on this host.  4 threads is what the
    reference uses (nth = 4, src/op.rs:1438); the all-core figure is reported beside it."""
    import oracle  # the CPU leg is the only place the benchmark touches the oracle
    ncpu = os.cpu_count() or 1
    try:
        ncpu = len(os.sched_getaffinity(0))
    except (AttributeError, OSError):
        pass
    res = {}
    total = sum(w.nbytes for w in weights_host)
    for label, nth in (("ref4", 4), ("all", max(1, min(ncpu, 64)))):
        # one untimed pass, then whole passes until the budget is used
        for (k, n), w in zip(GEMV_SHAPES, weights_host):
            oracle.cpu_mul_mat_q4_0_f32(w, xs_host[k], nth)
        t0 = time.perf_counter()
        passes = 0
        while True:
            for (k, n), w in zip(GEMV_SHAPES, weights_host):
                oracle.cpu_mul_mat_q4_0_f32(w, xs_host[k], nth)
            passes += 1
            dt = time.perf_counter() - t0
            if dt > budget_s or passes >= 20000:
                break
        res[label] = {"value": total * passes / dt / 1e9, "unit": "GB/s", "cores": nth, "kind": "port",
                      "sample": "%d passes over the 4-shape GEMV set (%.0f MB of Q4_0 weights per pass), %.1f s"
                                % (passes, total / 1e6, dt)}
    return res, ncpu


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--cpu-seconds", type=float, default=8.0, help="CPU baseline budget per thread setting")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-extra", action="store_true", help="skip prefill / row-kernel side measurements")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.stderr.write("bench.py: this build runs on ONE GPU (no collectives, no sharding); "
                         "--gpus %d is not supported, run with --gpus 1\n" % args.gpus)
        sys.exit(2)

    import galois_amd
    dev = galois_amd.Device(0)
    info = dev.info()
    rng = np.random.default_rng(0x9E3779B97F4A7C15 % (2 ** 63))

    # ---- inputs, resident in HBM before anything is timed
    base = [make_q4_matrix(dev, rng, k, n) for k, n in GEMV_SHAPES]
    set_bytes = sum(q4_bytes(k, n) for k, n in GEMV_SHAPES)
    nsets = max(2, -(-ROTATE_BYTES // set_bytes))
    sets = [base]
    for _ in range(nsets - 1):
        cp = []
        for (k, n), b in zip(GEMV_SHAPES, base):
            c = dev.alloc(q4_bytes(k, n))
            dev.copy_d2d(c, b, q4_bytes(k, n))
            cp.append(c)
        sets.append(cp)
    xs_host = {k: rng.standard_normal(k, dtype=np.float32) for k in (4096, 11008)}
    xs = {k: dev.upload(v) for k, v in xs_host.items()}
    ys = [dev.alloc(n * 4) for _, n in GEMV_SHAPES]
    dev.synchronize()

    def step(i):
        s = sets[i % nsets]
        for j, (k, n) in enumerate(GEMV_SHAPES):
            dev.dequantize_mul_mat_vec_q4_0(s[j], xs[k], ys[j], k, n)

    for i in range(args.warmup):
        step(i)
    ms = timed(dev, lambda i: step(i + args.warmup), args.steps)
    ms_per_step = ms / args.steps
    value = set_bytes / (ms_per_step * 1e-3) / 1e9
    launches = len(GEMV_SHAPES)
    avg_bytes = set_bytes / launches
    avg_us = ms_per_step * 1e3 / launches

    # per-shape figures (each shape alone, rotating over its own copies)
    per_shape = []
    for j, (k, n) in enumerate(GEMV_SHAPES):
        f = lambda i, j=j, k=k, n=n: dev.dequantize_mul_mat_vec_q4_0(sets[i % nsets][j], xs[k], ys[j], k, n)
        for i in range(20):
            f(i)
        us = timed(dev, f, 200, reps=5) / 200 * 1e3
        per_shape.append({"K": k, "N": n, "us": round(us, 3), "weight_GBps": round(q4_bytes(k, n) / us / 1e3, 1),
                          "hbm_frac": round(q4_bytes(k, n) / us / 1e3 / HBM_PEAK_GBPS, 4)})

    extra = {"device": info, "gemv_per_shape": per_shape, "rotating_weight_sets": nsets,
             "rotating_bytes": nsets * set_bytes}
    if not args.no_extra:
        m, k, n = PREFILL
        xp = dev.upload(rng.standard_normal((m, k), dtype=np.float32))
        yp = dev.alloc(m * n * 4)
        wp = base[1]  # K=4096 -> N=11008
        for _ in range(3):
            dev.mul_mat_q4_0_f32(wp, xp, yp, k, n, m)
        us = timed(dev, lambda i: dev.mul_mat_q4_0_f32(wp, xp, yp, k, n, m), 20, reps=5) / 20 * 1e3
        tf = 2.0 * m * k * n / us / 1e6
        extra["prefill_gemm"] = {"M": m, "K": k, "N": n, "us": round(us, 2), "TFLOPs": round(tf, 1),
                                 "roofline": {"bound": "mfma", "achieved": round(tf, 1),
                                              "peak": MFMA_F16_PEAK_TFLOPS, "unit": "TFLOP/s",
                                              "frac": round(tf / MFMA_F16_PEAK_TFLOPS, 4)}}
        # row kernels (configs[3]), algorithmic bytes from the byte table in DESIGN.md
        rows = {}
        a = dev.upload(rng.standard_normal((512, 4096), dtype=np.float32))
        b = dev.alloc(512 * 4096 * 4)
        g = dev.upload((1 + 0.1 * rng.standard_normal(4096)).astype(np.float32))
        us = timed(dev, lambda i: dev.rms_norm_mul_f32(a, g, b, 4096, 512, 1e-6), 100, reps=5) / 100 * 1e3
        rows["rms_norm_mul"] = {"us": round(us, 3), "GBps": round(16793600 / us / 1e3, 1)}
        pos = dev.upload(np.arange(512, dtype=np.int32))
        ts = float(np.float32(10000.0) ** np.float32(-2.0 / 128))
        us = timed(dev, lambda i: dev.rope_f32(a, b, 128, 512 * 32, pos, 1.0, 32, ts), 100, reps=5) / 100 * 1e3
        rows["rope"] = {"us": round(us, 3), "GBps": round(16779264 / us / 1e3, 1)}
        s = dev.upload((rng.standard_normal((32 * 512, 512), dtype=np.float32) * 3).astype(np.float32))
        so = dev.alloc(32 * 512 * 512 * 4)
        us = timed(dev, lambda i: dev.soft_max_causal_f32(s, so, 512, 512, 32 * 512, 0), 100, reps=5) / 100 * 1e3
        rows["soft_max_causal"] = {"us": round(us, 3), "GBps": round(50364416 / us / 1e3, 1)}
        for v in rows.values():
            v["hbm_frac"] = round(v["GBps"] / HBM_PEAK_GBPS, 4)
        extra["row_kernels"] = rows

    out = {
        "metric": "Q4_0 GEMV weight GB/s (% of HBM peak); Q4_0 prefill GEMM TFLOP/s @7B shapes",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 6), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "q4_0 x f32 (int4 dot, f32 scale)", "data": "synthetic",
        "config": {"workload": "LLaMA-7B-shaped Q4_0 GEMV set at batch 1: K4096->N4096, K4096->N11008, "
                               "K11008->N4096, K4096->N32000 (BASELINE.json configs[1])",
                   "weight_bytes_per_step": set_bytes, "launches_per_step": launches},
        "roofline": {"bound": "hbm", "achieved": round(avg_bytes / avg_us / 1e3, 1), "peak": HBM_PEAK_GBPS,
                     "unit": "GB/s", "frac": round(avg_bytes / avg_us / 1e3 / HBM_PEAK_GBPS, 4),
                     "traffic": GEMV_TRAFFIC_BYTES_PER_LAUNCH,
                     "kernel": "gemv_q4_0_dot8", "bytes_per_launch": avg_bytes, "us_per_launch": round(avg_us, 3)},
    }
    if not args.no_cpu:
        weights_host = [dev.download(b, np.uint8, (n, (k // 32) * 18)) for (k, n), b in zip(GEMV_SHAPES, base)]
        res, ncpu = cpu_baseline(weights_host, xs_host, args.cpu_seconds)
        out["cpu_baseline"] = res["ref4"]
        extra["cpu_baseline_all_cores"] = res["all"]
        extra["host_cpus_visible"] = ncpu
    out["extra"] = extra
    dev.close()
    print(json.dumps(out))


if __name__ == "__main__":
    main()
