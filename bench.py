#!/usr/bin/env python3
"""Benchmark of the Q4_0 hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

One step = one pass over the LLaMA-7B-shaped Q4_0 decode GEMV set at batch 1 (BASELINE.json
configs[1]): K=4096->N=4096, K=4096->N=11008, K=11008->N=4096, K=4096->N=32000, f32
activations N(0,1), weights N(0,0.02) quantized to Q4_0 on the device.  The four products of
a step go out as ONE grouped launch (galois_hip_dequantize_mul_mat_vec_q4_0_group: same
results, bit for bit, as four calls of the one-product entry point, which are timed beside it
under `extra`).  Successive steps rotate over distinct copies of the weights totalling more
than 1 GB so that every launch streams from HBM rather than from the 256 MB Infinity Cache.  Inputs are resident in HBM
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
# HBM bytes per grouped launch (the four products) measured with rocprofv3 --pmc FETCH_SIZE and WRITE_SIZE on
# this workload, each scaled by what the same counter reads for a device-to-device copy of known size
# (FETCH_SIZE x 1.9992, WRITE_SIZE x 1.000); see profiles/gemv_q4_0_group__llama7b_gemv_set.md
GEMV_TRAFFIC_BYTES_PER_LAUNCH = 135187713


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


SETTLE_S = 0.3   # every side measurement first runs its own launches for this long: after the idle time its set-up
                 # leaves (uploads, allocations) the device needs ~0.25 s of work to be back at its steady clocks
                 # (measured with rocm-smi: 1.4 -> 1.75 -> 1.9 -> 2.0 GHz over the first 0.3 s of a kernel loop), and a
                 # hundred launches of a 4-10 us kernel are over long before that


def settle(dev, fn, seconds=SETTLE_S):
    """Runs fn(i) back to back for `seconds` of wall time (synchronising every 64 calls)."""
    t_end = time.perf_counter() + seconds
    i = 0
    while time.perf_counter() < t_end:
        fn(i)
        i += 1
        if i % 64 == 0:
            dev.synchronize()
    dev.synchronize()
    return i


def timed(dev, fn, iters, reps=1, settle_s=0.0):
    """Median over `reps` of the event-timed duration (ms) of `iters` calls of fn(i)."""
    if settle_s:
        settle(dev, fn, settle_s)
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


USE_GRAPHS = True   # --no-graph: every graph-replay measurement falls back to eager launches (rocprofv3's kernel
                    # tracer does not survive thousands of graph launches)


def timed_graph(dev, fn, iters, reps=5, settle_s=0.0):
    """As timed(), with the `iters` launches recorded once into a HIP graph and replayed: the figure for kernels
    short enough that issuing them one by one from Python is what an eager loop measures."""
    if not USE_GRAPHS:
        return timed(dev, fn, iters, reps, settle_s)
    dev.synchronize()
    dev.graph_begin_capture()
    for i in range(iters):
        fn(i)
    graph = dev.graph_end_capture()
    e0, e1 = dev.event(), dev.event()
    dev.graph_launch(graph)
    if settle_s:
        settle(dev, lambda i: dev.graph_launch(graph), settle_s)
    out = []
    for _ in range(reps):
        dev.synchronize()
        dev.record(e0)
        dev.graph_launch(graph)
        dev.record(e1)
        out.append(dev.elapsed_ms(e0, e1))
    dev.synchronize()
    dev.graph_destroy(graph)
    dev.event_destroy(e0)
    dev.event_destroy(e1)
    return float(np.median(out))


def _host_cpus():
    try:
        return len(os.sched_getaffinity(0))
    except (AttributeError, OSError):
        return os.cpu_count() or 1


def _time_cpu(fn, budget_s, max_passes=20000):
    """One untimed pass, then whole passes until the budget is used: (passes, seconds)."""
    fn()
    t0 = time.perf_counter()
    passes = 0
    while True:
        fn()
        passes += 1
        dt = time.perf_counter() - t0
        if dt > budget_s or passes >= max_passes:
            return passes, dt


def cpu_baseline(weights_host, xs_host, budget_s):
    """The reference CPU op restated in C (oracle/), timed on this host.  4 threads is what the
    reference uses (nth = 4, src/op.rs:1438); the all-core figure is reported beside it."""
    import oracle  # the CPU leg is the only place the benchmark touches the oracle
    ncpu = _host_cpus()
    res = {}
    total = sum(w.nbytes for w in weights_host)

    def one_pass(nth):
        for (k, n), w in zip(GEMV_SHAPES, weights_host):
            oracle.cpu_mul_mat_q4_0_f32(w, xs_host[k], nth)

    for label, nth in (("ref4", 4), ("all", max(1, min(ncpu, 64)))):
        passes, dt = _time_cpu(lambda: one_pass(nth), budget_s)
        res[label] = {"value": total * passes / dt / 1e9, "unit": "GB/s", "cores": nth, "kind": "port",
                      "sample": "%d passes over the 4-shape GEMV set (%.0f MB of Q4_0 weights per pass), %.1f s"
                                % (passes, total / 1e6, dt)}
    return res, ncpu


def cpu_baseline_other_configs(w_4096x4096, w_4096x11008, x_vec, x_prefill, budget_s):
    """The same CPU op on BASELINE.json configs[0] (one 4096 x 4096 matvec) and configs[2] (the M = 512 prefill
    matmul, src/op.rs:1383-1598 with M > 1), each at the reference's 4 threads and at all cores."""
    import oracle
    ncpu = _host_cpus()
    out = {"single_matvec_4096x4096": {}, "prefill_512x4096x11008": {}}
    m, k, n = PREFILL
    for label, nth in (("ref4", 4), ("all", max(1, min(ncpu, 64)))):
        passes, dt = _time_cpu(lambda: oracle.cpu_mul_mat_q4_0_f32(w_4096x4096, x_vec, nth), budget_s)
        out["single_matvec_4096x4096"][label] = {
            "value": round(w_4096x4096.nbytes * passes / dt / 1e9, 2), "unit": "GB/s", "cores": nth, "kind": "port",
            "us_per_matvec": round(dt / passes * 1e6, 1), "sample": "%d matvecs, %.1f s" % (passes, dt)}
        passes, dt = _time_cpu(lambda: oracle.cpu_mul_mat_q4_0_f32(w_4096x11008, x_prefill, nth), budget_s)
        out["prefill_512x4096x11008"][label] = {
            "value": round(2.0 * m * k * n * passes / dt / 1e12, 4), "unit": "TFLOP/s", "cores": nth, "kind": "port",
            "ms_per_matmul": round(dt / passes * 1e3, 1), "sample": "%d matmuls of 512 x 4096 x 11008, %.1f s" % (passes, dt)}
    return out


def _normal_f32(seed, count, scale, threads=16):
    """count f32 draws of N(0, scale^2), generated by `threads` independent streams."""
    from concurrent.futures import ThreadPoolExecutor
    out = np.empty(count, np.float32)
    bounds = np.linspace(0, count, threads + 1).astype(np.int64)

    def fill(t):
        g = np.random.default_rng([seed, t])
        g.standard_normal(out=out[bounds[t]:bounds[t + 1]], dtype=np.float32)
        out[bounds[t]:bounds[t + 1]] *= np.float32(scale)

    with ThreadPoolExecutor(threads) as ex:
        list(ex.map(fill, range(threads)))
    return out


def decode_attention_bench(dev, rng):
    """The decode step's attention launches alone (BASELINE configs[4]'s shapes: 32 heads of 128, KV length 2048, f32
    caches): galois_hip_attn_decode_f32, and galois_hip_qkv_attn_decode_f32 with its three 4096 x 4096 products, over
    six copies of the caches in rotation (805 MB: no launch finds its rows in the Infinity Cache)."""
    H, D, L = 32, 128, 2048
    E = H * D
    nbuf = 6
    kcs = [dev.upload(rng.standard_normal((L, E), dtype=np.float32)) for _ in range(nbuf)]
    vcs = [dev.alloc(L * E * 4) for _ in range(nbuf)]
    for v_, k_ in zip(vcs, kcs[::-1]):
        dev.copy_d2d(v_, k_, L * E * 4)
    q, k, v = (dev.upload(rng.standard_normal(E, dtype=np.float32)) for _ in range(3))
    out = dev.alloc(E * 4)
    pos = dev.upload(np.array([L - 1], np.int32))
    ws = [make_q4_matrix(dev, rng, E, E) for _ in range(3)]
    x = dev.upload(rng.standard_normal(E, dtype=np.float32))
    items = dev.gemv_items([{"vx": w, "y": x, "dst": d, "ncols": E, "nrows": E} for w, d in zip(ws, (q, k, v))])
    ts = float(np.float32(10000.0) ** np.float32(-2.0 / D))
    cache_bytes = 2 * L * E * 4
    res = {}
    for name, f, nbytes in (
            ("attn_decode_f32", lambda i: dev.attn_decode_f32(q, k, v, kcs[i % nbuf], vcs[i % nbuf], out, H, D, L - 1, pos,
                                                              1.0, ts, D ** -0.5), cache_bytes),
            ("qkv_attn_decode_f32", lambda i: dev.qkv_attn_decode(items, kcs[i % nbuf], vcs[i % nbuf], out, H, D, L - 1,
                                                                   pos, 1.0, ts, D ** -0.5), cache_bytes + 3 * q4_bytes(E, E))):
        us = timed_graph(dev, f, 60, settle_s=SETTLE_S) / 60 * 1e3
        res[name] = {"us": round(us, 3), "algorithmic_bytes": nbytes, "GBps": round(nbytes / us / 1e3, 1),
                     "hbm_frac": round(nbytes / us / 1e3 / HBM_PEAK_GBPS, 4)}
    for b_ in kcs + vcs + ws + [q, k, v, out, pos, x]:
        dev.free(b_)
    return res


def prefill_attention_bench(dev, rng):
    """Causal attention of 512 rows for 32 heads of 128 in one launch (galois_hip_attn_prefill_*), writing the fp16
    panel of the output projection: an empty context and a context of 1536 positions, f32 and f16 caches.  The caches
    rotate over six copies.  flop = the two products under the mask (4 * head_dim per visible (query, key) pair)."""
    H, D, n = 32, 128, 512
    E = H * D
    res = {}
    q = dev.upload(rng.standard_normal((n, E), dtype=np.float32))
    panel = dev.alloc(dev.f16_panel_bytes(E, n))
    for n_past in (0, 1536):
        L = n_past + n
        for kv_f16 in (False, True):
            nbuf = 6 if n_past == 0 else 3
            host = rng.standard_normal((L, E), dtype=np.float32)
            host = host.astype(np.float16) if kv_f16 else host
            kcs = [dev.upload(host) for _ in range(nbuf)]
            vcs = [dev.upload(host) for _ in range(nbuf)]
            f = lambda i: dev.attn_prefill(q, kcs[i % nbuf], vcs[i % nbuf], None, panel, H, D, n, n_past, D ** -0.5, kv_f16)
            us = timed_graph(dev, f, 60, settle_s=SETTLE_S) / 60 * 1e3
            flop = 4.0 * D * H * sum(n_past + m + 1 for m in range(n))
            res["n_past_%d_%s_cache" % (n_past, "f16" if kv_f16 else "f32")] = {
                "us": round(us, 2), "TFLOPs_under_the_mask": round(flop / us / 1e6, 1),
                "cache_bytes": 2 * L * E * (2 if kv_f16 else 4)}
            for b_ in kcs + vcs:
                dev.free(b_)
    dev.free(q)
    dev.free(panel)
    return res


SETTLE_STEPS = 150   # decode steps (1.6-3 ms each) run before a plan is timed: the same settling as SETTLE_S


def decode_step_bench(dev, reps, with_graph=True, prefill_only=False):
    """BASELINE.json configs[4]: a 32-layer LLaMA-7B-architecture decode step at KV length 2048, issued through the
    host mirror's galois ops, random-init weights quantized on the device.  Returns tokens/s three ways."""
    from galois_amd import host_api as g
    t0 = time.time()
    gdev = g.Device.gpu(0)
    seed = [0]

    def make_decoder(kv_f16, head_major=False):
        seed[0] = 0   # every decoder gets the same weights and the same cache contents
        dec = g.LlamaDecoder(gdev, kv_f16=kv_f16, kv_head_major=head_major)   # defaults = the config: 4096 / 32 heads / 11008 / 32000 / 32 layers
        hp = dec.hp
        e, f, v, c = hp["n_embd"], hp["n_ff"], hp["n_vocab"], hp["n_ctx"]
        stage = dev.alloc(e * v * 4)

        def fill_q4(t, rows, cols):
            seed[0] += 1
            dev.upload(_normal_f32(seed[0], rows * cols, 0.02), stage)
            dev.quantize_row_q4_0(stage, t.data_ptr(), rows * cols)
            dev.synchronize()

        def fill_f32(t, count, mean, scale, f16=False, cache=False):
            seed[0] += 1
            a = _normal_f32(seed[0], count, scale) + np.float32(mean)
            if cache and head_major:   # the same elements, kept [n_head][n_ctx][head_dim]
                a = np.ascontiguousarray(a.reshape(c, hp["n_head"], -1).transpose(1, 0, 2)).ravel()
            t.write(a.astype(np.float16) if f16 else a)

        fill_q4(dec.tensor("tok_embd"), v, e)
        fill_q4(dec.tensor("output"), v, e)
        fill_f32(dec.tensor("out_norm"), e, 1.0, 0.1)
        weight_bytes = q4_bytes(e, v)               # the embedding table is read one row per token
        for i in range(hp["n_layer"]):
            for n, rows, cols in (("wq", e, e), ("wk", e, e), ("wv", e, e), ("wo", e, e), ("w_gate", f, e),
                                  ("w_up", f, e), ("w_down", e, f)):
                fill_q4(dec.tensor(n, i), rows, cols)
                weight_bytes += q4_bytes(cols, rows)
            fill_f32(dec.tensor("attn_norm", i), e, 1.0, 0.1)
            fill_f32(dec.tensor("ffn_norm", i), e, 1.0, 0.1)
            fill_f32(dec.tensor("k_cache", i), e * c, 0.0, 1.0, kv_f16, True)
            fill_f32(dec.tensor("v_cache", i), e * c, 0.0, 1.0, kv_f16, True)
        dev.free(stage)
        return dec, weight_bytes

    dec, weight_bytes = make_decoder(False)
    hp = dec.hp
    e, c = hp["n_embd"], hp["n_ctx"]
    kv_bytes = hp["n_layer"] * 2 * c * e * 4
    setup_s = time.time() - t0
    tok, n_past = 1, c - 1
    res = {"config": "32 layers, d_model 4096, 32 heads, FFN 11008, vocab 32000, KV length %d, f32 cache" % c,
           "algorithmic_bytes_per_token": weight_bytes + kv_bytes, "setup_s": round(setup_s, 1)}
    plan_logits = {}

    def cross(a, b):  # max |a - b| / max |b| and relative L2 of two sets of logits
        return {"max_rel": float(np.max(np.abs(a - b)) / np.max(np.abs(b))),
                "l2_rel": float(np.linalg.norm(a - b) / np.linalg.norm(b))}

    def prefill(dec, n_tok=512, compare=True):
        """n_tok tokens from an empty context in one pass (LlamaDecoder.prefill: the Q4_0 products through the prefill
        matmul on fp16 panels) against the same tokens decoded one by one on the same decoder."""
        hp = dec.hp
        e, f = hp["n_embd"], hp["n_ff"]
        toks = np.random.default_rng(11).integers(0, hp["n_vocab"], n_tok).astype(np.int32)
        if compare:
            t_dec = time.time()
            for i, t in enumerate(toks):
                dec.decode(int(t), i, 5)
            one_by_one = dec.logits().astype(np.float64)     # (the download waits for the stream)
            ms_one_by_one = (time.time() - t_dec) * 1e3
        dec.prefill(toks, 0)
        got = dec.logits().astype(np.float64)
        dec.time_prefill(toks, 0, 4)
        ms = min(dec.time_prefill(toks, 0, 4) for _ in range(3)) / 4
        q4_flop = 2.0 * n_tok * hp["n_layer"] * (4 * e * e + 3 * e * f)
        attn_flop = 2.0 * 2 * n_tok * n_tok * e * hp["n_layer"]     # scores and out over all n_tok keys (the masked half too)
        if not compare:
            return {"tokens": n_tok, "library_calls": dec.ops_per_prefill(), "ms": round(ms, 3), "tokens_per_s": round(n_tok / ms * 1e3, 0),
                    "q4_0_flop_over_the_whole_pass_TFLOPs": round(q4_flop / ms / 1e9, 1),
                    "q4_0_flop_over_the_whole_pass_mfma_frac": round(q4_flop / ms / 1e9 / MFMA_F16_PEAK_TFLOPS, 4),
                    "logits_finite": bool(np.all(np.isfinite(got)))}
        return {"tokens": n_tok, "library_calls": dec.ops_per_prefill(), "ms": round(ms, 3), "tokens_per_s": round(n_tok / ms * 1e3, 0),
                "q4_0_flop_over_the_whole_pass_TFLOPs": round(q4_flop / ms / 1e9, 1),
                "q4_0_flop_over_the_whole_pass_mfma_frac": round(q4_flop / ms / 1e9 / MFMA_F16_PEAK_TFLOPS, 4),
                "q4_0_flop": q4_flop, "attention_flop": attn_flop,
                "ms_decoding_one_by_one": round(ms_one_by_one, 1), "speedup_over_decoding_one_by_one": round(ms_one_by_one / ms, 1),
                "last_logits_vs_one_by_one": cross(got, one_by_one)}

    if prefill_only:
        res["prefill_512_tokens"] = prefill(dec)
        dec.close()
        return res
    for name, fused in (("eager_one_kernel_per_op", 0), ("eager_fused_norm_and_silu", 1), ("eager_grouped_gemv", 2),
                        ("eager_grouped_gemv_fused_attention", 3), ("eager_split_norms", 4),
                        ("eager_qkv_and_attention_in_one_launch", 5)):
        dec.time_steps(tok, n_past, fused, SETTLE_STEPS)
        ms = min(dec.time_steps(tok, n_past, fused, reps) for _ in range(3)) / reps
        res[name] = {"launches": dec.ops_per_step(), "ms_per_token": round(ms, 4), "tokens_per_s": round(1e3 / ms, 1)}
        plan_logits[fused] = dec.logits().astype(np.float64)
    if not with_graph:
        res["prefill_512_tokens"] = prefill(dec)
        dec.close()
        return res
    graph_logits = {}
    for name, fused in (("hip_graph_split_norms", 4), ("hip_graph_qkv_and_attention_in_one_launch", 5)):
        dec.capture(tok, n_past, fused)
        dec.time_replays(SETTLE_STEPS)
        ms = min(dec.time_replays(reps) for _ in range(3)) / reps
        res[name] = {"launches": dec.ops_per_step(), "ms_per_token": round(ms, 4), "tokens_per_s": round(1e3 / ms, 1),
                     "GBps": round((weight_bytes + kv_bytes) / ms / 1e6, 1),
                     "hbm_frac": round((weight_bytes + kv_bytes) / ms / 1e6 / HBM_PEAK_GBPS, 4)}
        graph_logits[name] = dec.logits().astype(np.float64)
    logits = dec.logits()
    res["logits_finite"] = bool(np.all(np.isfinite(logits)))
    # the 32-layer logits of the fused plans and of the graph replay against the one-kernel-per-op plan (every op its
    # own launch, each of them parity-tested against the oracle at these shapes): the bar is the matvec's 1e-4
    res["logits_vs_one_kernel_per_op"] = {
        "grouped_gemv_fused_attention": cross(plan_logits[3], plan_logits[0]),
        "split_norms": cross(plan_logits[4], plan_logits[0]),
        "qkv_and_attention_in_one_launch": cross(plan_logits[5], plan_logits[0]),
        **{k: cross(v, plan_logits[0]) for k, v in graph_logits.items()}}
    res["logits_within_1e-4"] = bool(all(v["max_rel"] < 1e-4 and v["l2_rel"] < 1e-4
                                         for v in res["logits_vs_one_kernel_per_op"].values()))
    res["prefill_512_tokens"] = prefill(dec)
    res["prefill_2048_tokens"] = prefill(dec, 2048, compare=False)   # a whole context in one pass
    dec.close()
    # the same step with the caches kept [n_head][n_ctx][head_dim]: a head's keys contiguous (same weights, same cache
    # contents: the logits are compared with the one-kernel-per-op plan of the [n_ctx][n_embd] decoder above)
    dec, _ = make_decoder(False, True)
    for name, fused in (("eager_split_norms_head_major_kv", 4), ("eager_qkv_and_attention_in_one_launch_head_major_kv", 5)):
        dec.time_steps(tok, n_past, fused, SETTLE_STEPS)
        ms = min(dec.time_steps(tok, n_past, fused, reps) for _ in range(3)) / reps
        res[name] = {"launches": dec.ops_per_step(), "ms_per_token": round(ms, 4), "tokens_per_s": round(1e3 / ms, 1),
                     "GBps": round((weight_bytes + kv_bytes) / ms / 1e6, 1),
                     "hbm_frac": round((weight_bytes + kv_bytes) / ms / 1e6 / HBM_PEAK_GBPS, 4),
                     "logits_vs_one_kernel_per_op": cross(dec.logits().astype(np.float64), plan_logits[0])}
    dec.close()
    # the same step with the KV cache in f16 (the form the reference keeps it in on the GPU): half the cache bytes
    dec, _ = make_decoder(True)
    b16 = weight_bytes + kv_bytes // 2
    for name, fused in (("eager_split_norms_f16_kv", 4), ("eager_qkv_and_attention_in_one_launch_f16_kv", 5)):
        dec.time_steps(tok, n_past, fused, SETTLE_STEPS)
        ms = min(dec.time_steps(tok, n_past, fused, reps) for _ in range(3)) / reps
        res[name] = {
            "launches": dec.ops_per_step(), "ms_per_token": round(ms, 4), "tokens_per_s": round(1e3 / ms, 1),
            "algorithmic_bytes_per_token": b16, "GBps": round(b16 / ms / 1e6, 1),
            "hbm_frac": round(b16 / ms / 1e6 / HBM_PEAK_GBPS, 4),
            "logits_finite": bool(np.all(np.isfinite(dec.logits())))}
    res["prefill_512_tokens_f16_kv"] = prefill(dec)
    dec.close()
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="CPU baseline budget per thread setting")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-extra", action="store_true", help="skip prefill / row-kernel side measurements")
    ap.add_argument("--no-decode", action="store_true", help="skip the 32-layer decode-step measurement")
    ap.add_argument("--prefill-only", action="store_true",
                    help="of the 32-layer measurements only the 512-token prefill pass (f32 caches); for runs under the tracer")
    ap.add_argument("--decode-no-graph", action="store_true",
                    help="decode step: eager launches only (graph replays cannot run under the kernel tracer)")
    ap.add_argument("--no-graph", action="store_true",
                    help="no HIP-graph replays anywhere: graph figures are measured as eager launches (for runs under "
                         "rocprofv3 --kernel-trace); implies --decode-no-graph")
    args = ap.parse_args()
    global USE_GRAPHS
    if args.no_graph:
        USE_GRAPHS = False
        args.decode_no_graph = True
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

    groups = [dev.gemv_items([{"vx": s[j], "y": xs[k], "dst": ys[j], "ncols": k, "nrows": n}
                              for j, (k, n) in enumerate(GEMV_SHAPES)]) for s in sets]

    def step(i):  # the four products of the set in one launch
        dev.dequantize_mul_mat_vec_q4_0_group(groups[i % nsets])

    def step_separate(i):  # one launch per product, as the reference issues them (src/cuda.rs:1026-1034)
        s = sets[i % nsets]
        for j, (k, n) in enumerate(GEMV_SHAPES):
            dev.dequantize_mul_mat_vec_q4_0(s[j], xs[k], ys[j], k, n)

    # Before the W warm-up steps the device is brought to its steady state (clocks, TLB entries of the 1.3 GB of
    # rotating weights): measured, the first ~50 ms of launches after an idle period run about 10 % slower.
    t_end = time.perf_counter() + 0.25
    i = 0
    while time.perf_counter() < t_end:
        step(i)
        i += 1
        if i % 256 == 0:
            dev.synchronize()
    dev.synchronize()
    for i in range(args.warmup):
        step(i)
    ms = timed(dev, lambda i: step(i + args.warmup), args.steps)
    ms_per_step = ms / args.steps
    value = set_bytes / (ms_per_step * 1e-3) / 1e9
    launches = 1
    avg_bytes = set_bytes / launches
    avg_us = ms_per_step * 1e3 / launches
    for i in range(args.warmup):
        step_separate(i)
    ms_sep = timed(dev, step_separate, args.steps) / args.steps

    # per-shape figures (each shape alone, rotating over its own copies)
    per_shape = []
    for j, (k, n) in enumerate(GEMV_SHAPES):
        f = lambda i, j=j, k=k, n=n: dev.dequantize_mul_mat_vec_q4_0(sets[i % nsets][j], xs[k], ys[j], k, n)
        for i in range(20):
            f(i)
        us = timed(dev, f, 200, reps=5, settle_s=SETTLE_S) / 200 * 1e3
        us_graph = timed_graph(dev, f, 200, settle_s=SETTLE_S) / 200 * 1e3   # the same launches replayed from a HIP graph: no host in the loop
        per_shape.append({"K": k, "N": n, "us": round(us, 3), "us_graph_replay": round(us_graph, 3),
                          "weight_GBps": round(q4_bytes(k, n) / us / 1e3, 1),
                          "hbm_frac": round(q4_bytes(k, n) / us / 1e3 / HBM_PEAK_GBPS, 4)})

    extra = {"device": info,
             "one_launch_per_product": {"ms_per_step": round(ms_sep, 6), "launches_per_step": len(GEMV_SHAPES),
                                        "weight_GBps": round(set_bytes / ms_sep / 1e6, 1),
                                        "hbm_frac": round(set_bytes / ms_sep / 1e6 / HBM_PEAK_GBPS, 4)},
             "gemv_per_shape": per_shape, "rotating_weight_sets": nsets, "rotating_bytes": nsets * set_bytes}
    if not args.no_extra:
        m, k, n = PREFILL
        xp = dev.upload(rng.standard_normal((m, k), dtype=np.float32))
        yp = dev.alloc(m * n * 4)
        wp = base[1]  # K=4096 -> N=11008
        for _ in range(50):  # warm: the fp16 workspace is allocated on the first call, clocks settle
            dev.mul_mat_q4_0_f32(wp, xp, yp, k, n, m)
        us = timed(dev, lambda i: dev.mul_mat_q4_0_f32(wp, xp, yp, k, n, m), 100, reps=5, settle_s=SETTLE_S) / 100 * 1e3
        tf = 2.0 * m * k * n / us / 1e6
        extra["prefill_gemm"] = {"M": m, "K": k, "N": n, "us": round(us, 2), "TFLOPs": round(tf, 1),
                                 "roofline": {"bound": "mfma", "achieved": round(tf, 1),
                                              "peak": MFMA_F16_PEAK_TFLOPS, "unit": "TFLOP/s",
                                              "frac": round(tf / MFMA_F16_PEAK_TFLOPS, 4)}}
        # the other prefill shapes of a LLaMA-7B layer (narrow matrices take the 256 x 48 tile)
        others = []
        for (k2, n2), wq in ((GEMV_SHAPES[0], base[0]), (GEMV_SHAPES[2], base[2])):
            xo = dev.upload(rng.standard_normal((m, k2), dtype=np.float32))
            yo = dev.alloc(m * n2 * 4)
            for _ in range(20):
                dev.mul_mat_q4_0_f32(wq, xo, yo, k2, n2, m)
            uso = timed(dev, lambda i: dev.mul_mat_q4_0_f32(wq, xo, yo, k2, n2, m), 50, reps=5, settle_s=SETTLE_S) / 50 * 1e3
            others.append({"M": m, "K": k2, "N": n2, "us": round(uso, 2), "TFLOPs": round(2.0 * m * k2 * n2 / uso / 1e6, 1)})
            dev.free(xo)
            dev.free(yo)
        extra["prefill_gemm_other_shapes"] = others
        # The same matmul on activations that are already an fp16 panel (written once by the op that produces them:
        # a conversion, an RMSNorm or a SwiGLU), and several matrices of a layer against one panel in one launch.  These
        # are NOT the configs[2] figure above (there X is f32 and is converted inside the timed call); they are what a
        # prefill graph built on the panel calls sees.
        pb = dev.alloc(dev.f16_panel_bytes(k, m))
        dev.f32_to_f16_panel(xp, pb, k, m)
        gnorm = dev.upload((1 + 0.1 * rng.standard_normal(k)).astype(np.float32))
        w3 = [base[0]] + [dev.alloc(q4_bytes(4096, 4096)) for _ in range(2)]
        for c in w3[1:]:
            dev.copy_d2d(c, base[0], q4_bytes(4096, 4096))
        w2 = [wp, sets[1][1]]
        y3 = [dev.alloc(m * 4096 * 4) for _ in range(3)]
        y2 = [yp, dev.alloc(m * n * 4)]
        panel = {}

        def tpanel(name, fn, flop, calls=50):
            for _ in range(20):
                fn()
            usp = timed(dev, lambda i: fn(), calls, reps=5, settle_s=SETTLE_S) / calls * 1e3
            panel[name] = {"us": round(usp, 2)}
            if flop:
                panel[name].update(TFLOPs=round(flop / usp / 1e6, 1), mfma_frac=round(flop / usp / 1e6 / MFMA_F16_PEAK_TFLOPS, 4))

        tpanel("f32_to_panel_512x4096", lambda: dev.f32_to_f16_panel(xp, pb, k, m), 0)
        tpanel("rms_norm_mul_to_panel_512x4096", lambda: dev.rms_norm_mul_f16_panel(xp, gnorm, pb, k, m, 1e-6), 0)
        dev.f32_to_f16_panel(xp, pb, k, m)
        tpanel("matmul_512x4096x11008", lambda: dev.mul_mat_q4_0_f16_panel([(wp, yp, n)], pb, k, m), 2.0 * m * k * n)
        tpanel("gate_up_one_launch_512x4096x2x11008",
               lambda: dev.mul_mat_q4_0_f16_panel([(w, y, n) for w, y in zip(w2, y2)], pb, k, m), 2 * 2.0 * m * k * n)
        pf2 = dev.alloc(dev.f16_panel_bytes(n, m))
        tpanel("gate_up_one_launch_then_swiglu_to_panel",
               lambda: (dev.mul_mat_q4_0_f16_panel([(w, y, n) for w, y in zip(w2, y2)], pb, k, m),
                        dev.silu_mul_f16_panel(y2[0], y2[1], pf2, n, m)), 2 * 2.0 * m * k * n)
        tpanel("gate_up_and_swiglu_one_launch_512x4096x2x11008",
               lambda: dev.mul_mat_q4_0_swiglu_f16_panel(w2[0], w2[1], pb, pf2, k, n, m), 2 * 2.0 * m * k * n)
        dev.free(pf2)
        tpanel("qkv_one_launch_512x4096x3x4096",
               lambda: dev.mul_mat_q4_0_f16_panel([(w, y, 4096) for w, y in zip(w3, y3)], pb, k, m), 3 * 2.0 * m * k * 4096)
        tpanel("qkv_three_f32_calls_512x4096x4096",
               lambda: [dev.mul_mat_q4_0_f32(w, xp, y, k, 4096, m) for w, y in zip(w3, y3)], 3 * 2.0 * m * k * 4096)
        # an output / down projection with the residual added: the plain product and the add, against the call that
        # folds them (with a workspace a narrow matrix runs as two shares of k)
        kd, nd = 11008, 4096
        wdn = make_q4_matrix(dev, rng, kd, nd)
        xd = dev.upload(rng.standard_normal((m, kd), dtype=np.float32))
        pd = dev.alloc(dev.f16_panel_bytes(kd, m))
        dev.f32_to_f16_panel(xd, pd, kd, m)
        res_b, yd, y2d, wsd = dev.upload(rng.standard_normal((m, nd), dtype=np.float32)), dev.alloc(m * nd * 4), dev.alloc(m * nd * 4), dev.alloc(2 * m * nd * 4)
        tpanel("down_512x11008x4096_then_add",
               lambda: (dev.mul_mat_q4_0_f16_panel([(wdn, yd, nd)], pd, kd, m), dev.add_f32(yd, res_b, y2d, m * nd, m * nd)), 2.0 * m * kd * nd)
        tpanel("down_512x11008x4096_with_residual_two_shares_of_k",
               lambda: dev.mul_mat_q4_0_f16_panel_add(wdn, pd, res_b, y2d, kd, nd, m, wsd, 2 * m * nd * 4), 2.0 * m * kd * nd)
        tpanel("out_512x4096x4096_then_add",
               lambda: (dev.mul_mat_q4_0_f16_panel([(w3[0], yd, nd)], pb, k, m), dev.add_f32(yd, res_b, y2d, m * nd, m * nd)), 2.0 * m * k * nd)
        tpanel("out_512x4096x4096_with_residual_two_shares_of_k",
               lambda: dev.mul_mat_q4_0_f16_panel_add(w3[0], pb, res_b, y2d, k, nd, m, wsd, 2 * m * nd * 4), 2.0 * m * k * nd)
        for b_ in (wdn, xd, pd, res_b, yd, y2d, wsd):
            dev.free(b_)
        extra["prefill_gemm_fp16_panel"] = panel
        for b_ in [pb, gnorm, y2[1]] + w3[1:] + y3:
            dev.free(b_)
        # row kernels (configs[3]); algorithmic bytes: rms_norm + weight = read + write of 512 x 4096 f32 + the weight
        # row, rope = read + write + positions, causal softmax = lower triangle read + full write of 32 x 512 x 512 f32
        # Inputs and outputs rotate over enough copies (> 256 MB in total) that no launch finds its rows in the
        # Infinity Cache; 100 launches are replayed from a HIP graph (issued one by one from Python the two short
        # kernels are bound by the interpreter: that figure is kept beside it as us_eager).
        rows = {}
        nrot = 10
        a_host = rng.standard_normal((512, 4096), dtype=np.float32)
        ins = [dev.upload(a_host) for _ in range(nrot)]
        outs = [dev.alloc(512 * 4096 * 4) for _ in range(nrot)]
        g = dev.upload((1 + 0.1 * rng.standard_normal(4096)).astype(np.float32))
        f = lambda i: dev.rms_norm_mul_f32(ins[i % nrot], g, outs[i % nrot], 4096, 512, 1e-6)
        us = timed_graph(dev, f, 100, settle_s=SETTLE_S) / 100 * 1e3
        rows["rms_norm_mul"] = {"us": round(us, 3), "GBps": round(16793600 / us / 1e3, 1),
                                "us_eager": round(timed(dev, f, 100, reps=5) / 100 * 1e3, 3)}
        pos = dev.upload(np.arange(512, dtype=np.int32))
        ts = float(np.float32(10000.0) ** np.float32(-2.0 / 128))
        f = lambda i: dev.rope_f32(ins[i % nrot], outs[i % nrot], 128, 512 * 32, pos, 1.0, 32, ts)
        us = timed_graph(dev, f, 100, settle_s=SETTLE_S) / 100 * 1e3
        rows["rope"] = {"us": round(us, 3), "GBps": round(16779264 / us / 1e3, 1),
                        "us_eager": round(timed(dev, f, 100, reps=5) / 100 * 1e3, 3)}
        for b_ in ins + outs:
            dev.free(b_)
        nrot = 4                                             # 4 x (33.5 MB in + 33.5 MB out)
        s_host = (rng.standard_normal((32 * 512, 512), dtype=np.float32) * 3).astype(np.float32)
        sin = [dev.upload(s_host) for _ in range(nrot)]
        sout = [dev.alloc(32 * 512 * 512 * 4) for _ in range(nrot)]
        f = lambda i: dev.soft_max_causal_f32(sin[i % nrot], sout[i % nrot], 512, 512, 32 * 512, 0)
        us = timed_graph(dev, f, 100, settle_s=SETTLE_S) / 100 * 1e3
        rows["soft_max_causal"] = {"us": round(us, 3), "GBps": round(50364416 / us / 1e3, 1),
                                   "us_eager": round(timed(dev, f, 100, reps=5) / 100 * 1e3, 3)}
        for b_ in sin + sout:
            dev.free(b_)
        for v in rows.values():
            v["hbm_frac"] = round(v["GBps"] / HBM_PEAK_GBPS, 4)
        extra["row_kernels"] = rows
        extra["decode_attention"] = decode_attention_bench(dev, rng)
        extra["prefill_attention"] = prefill_attention_bench(dev, rng)

    out = {
        "metric": "Q4_0 GEMV weight GB/s (% of HBM peak); Q4_0 prefill GEMM TFLOP/s @7B shapes",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 6), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "q4_0 x f32 (int4 dot, f32 scale)", "data": "synthetic",
        "config": {"workload": "LLaMA-7B-shaped Q4_0 GEMV set at batch 1: K4096->N4096, K4096->N11008, "
                               "K11008->N4096, K4096->N32000 (BASELINE.json configs[1]), the four products in one "
                               "grouped launch",
                   "weight_bytes_per_step": set_bytes, "launches_per_step": launches},
        "roofline": {"bound": "hbm", "achieved": round(avg_bytes / avg_us / 1e3, 1), "peak": HBM_PEAK_GBPS,
                     "unit": "GB/s", "frac": round(avg_bytes / avg_us / 1e3 / HBM_PEAK_GBPS, 4),
                     "traffic": GEMV_TRAFFIC_BYTES_PER_LAUNCH,
                     "traffic_source": "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this command, summarised in "
                                       "profiles/gemv_q4_0_group__llama7b_gemv_set.md (a constant from that profile, "
                                       "not measured in this run)",
                     "kernel": "gemv_q4_0_group", "bytes_per_launch": avg_bytes, "us_per_launch": round(avg_us, 3)},
    }
    if not args.no_decode:
        extra["decode_step"] = decode_step_bench(dev, 10, not args.decode_no_graph, args.prefill_only)
    if not args.no_cpu:
        weights_host = [dev.download(b, np.uint8, (n, (k // 32) * 18)) for (k, n), b in zip(GEMV_SHAPES, base)]
        res, ncpu = cpu_baseline(weights_host, xs_host, args.cpu_seconds)
        out["cpu_baseline"] = res["ref4"]
        extra["cpu_baseline_all_cores"] = res["all"]
        extra["host_cpus_visible"] = ncpu
        x_prefill = np.random.default_rng(5).standard_normal((PREFILL[0], PREFILL[1]), dtype=np.float32)
        extra["cpu_baseline_other_configs"] = cpu_baseline_other_configs(
            weights_host[0], weights_host[1], xs_host[4096], x_prefill, max(1.0, args.cpu_seconds / 4))
    out["extra"] = extra
    dev.close()
    print(json.dumps(out))


if __name__ == "__main__":
    main()
