"""The launch that carries the q | k | v products and the decode attention together against the same two calls issued
one after the other.  q, k, v and the appended cache rows are bit-equal whenever the products' own call runs the same
workgroup shape (8 waves x 2 rows); with few rows it runs 16 waves x 1 row, which adds up a normalising product's
sum of squares in another order, so there the bar is 2e-6 of the largest element.  The attention's output agrees up to
the order of its f32 sums (eight waves instead of four share a split's keys): 1e-5 of the largest output, the
tolerance of the attention's own parity test."""
import numpy as np
import pytest

import oracle

pytestmark = pytest.mark.gpu


def _case(dev, H, K, n_past, mode, kv_f16, seed, repeats=1, n_ctx=None):
    D = 128
    E = H * D
    rng = np.random.default_rng(seed)
    n_ctx = n_ctx or n_past + 1
    ws = [dev.upload(oracle.quantize_q4_0((rng.standard_normal((E, K)) * 0.05).astype(np.float32))) for _ in range(3)]
    x = dev.upload(rng.standard_normal(K).astype(np.float32))
    nw = dev.upload((1 + 0.1 * rng.standard_normal(K)).astype(np.float32))
    ssq = dev.upload(np.abs(rng.standard_normal((K + 15) // 16)).astype(np.float32) * 16)
    ct = np.float16 if kv_f16 else np.float32
    kc0 = rng.standard_normal((n_ctx, E)).astype(ct)
    vc0 = rng.standard_normal((n_ctx, E)).astype(ct)
    pos = dev.upload(np.array([n_past], np.int32))
    fs, ts, scale = 1.0, 10000.0 ** (-2.0 / D), D ** -0.5

    def side():
        q, k, v = (dev.upload(np.full(E, 3.25, np.float32)) for _ in range(3))
        items = []
        for w, d in zip(ws, (q, k, v)):
            it = {"vx": w, "y": x, "dst": d, "ncols": K, "nrows": E}
            if mode == 1:
                it.update(norm_weight=nw, norm_eps=1e-5)
            elif mode == 2:
                it.update(sumsq_in=ssq, norm_eps=1e-5)
            items.append(it)
        return dict(q=q, k=k, v=v, items=dev.gemv_items(items), kc=dev.upload(kc0), vc=dev.upload(vc0),
                    out=dev.upload(np.full(E + 16, 7.5, np.float32)))

    a, b = side(), side()
    for r in range(repeats):
        print("qkv_attn case H=%d K=%d n_past=%d mode=%d f16=%s rep=%d" % (H, K, n_past, mode, kv_f16, r), flush=True)
        dev.dequantize_mul_mat_vec_q4_0_group(a["items"])
        attn = dev.attn_decode_f16kv if kv_f16 else dev.attn_decode_f32
        attn(a["q"], a["k"], a["v"], a["kc"], a["vc"], a["out"], H, D, n_past, pos, fs, ts, scale)
        dev.qkv_attn_decode(b["items"], b["kc"], b["vc"], b["out"], H, D, n_past, pos, fs, ts, scale, kv_f16=kv_f16)
        dev.synchronize()
        for name, n, t in (("q", E, np.float32), ("k", E, np.float32), ("v", E, np.float32), ("out", E + 16, np.float32),
                           ("kc", kc0.shape, ct), ("vc", vc0.shape, ct)):
            ra, rb = dev.download(a[name], t, n), dev.download(b[name], t, n)
            if name == "out":
                assert np.all(np.isfinite(rb[:E])) and np.all(rb[E:] == 7.5)
                assert np.max(np.abs(ra[:E] - rb[:E])) <= 1e-5 * np.max(np.abs(ra[:E])), r
            elif 3 * E > 16 * 256:   # more than 16 rows per CU: the products' own call runs the same workgroup shape
                assert np.array_equal(ra.view(np.uint8), rb.view(np.uint8)), (name, r)
            else:
                fa, fb = ra.astype(np.float32), rb.astype(np.float32)
                assert np.max(np.abs(fa - fb)) <= (1e-3 if kv_f16 else 2e-6) * np.max(np.abs(fa)), (name, r)
    for s in (a, b):
        for key in ("q", "k", "v", "kc", "vc", "out"):
            dev.free(s[key])
    for buf in ws + [x, nw, ssq, pos]:
        dev.free(buf)


@pytest.mark.parametrize("H,K,n_past,mode,kv_f16", [
    (2, 256, 0, 0, False), (2, 256, 5, 1, False), (3, 320, 130, 2, False), (4, 256, 127, 1, True),
    (2, 5120, 300, 1, False), (2, 4160, 300, 2, True), (2, 4160, 40, 0, False), (2, 11776, 70, 1, False),
    (32, 4096, 2047, 2, False), (32, 4096, 2047, 1, False), (32, 4096, 2047, 2, True), (32, 4096, 2300, 0, False)])
def test_qkv_attn_equals_the_two_calls(dev, H, K, n_past, mode, kv_f16):
    _case(dev, H, K, n_past, mode, kv_f16, seed=H * 1000 + n_past)


@pytest.mark.parametrize("H,K,n_past,n_ctx,kv_f16", [(32, 4096, 2047, 2048, False), (3, 256, 130, 200, True)])
def test_qkv_attn_with_head_major_caches(dev, H, K, n_past, n_ctx, kv_f16):
    """The same launch over caches kept [n_head][n_ctx][head_dim]: outputs and cache contents bit-equal."""
    D = 128
    E = H * D
    rng = np.random.default_rng(H + n_past)
    ct = np.float16 if kv_f16 else np.float32
    ws = [dev.upload(oracle.quantize_q4_0((rng.standard_normal((E, K)) * 0.05).astype(np.float32))) for _ in range(3)]
    x, nw = dev.upload(rng.standard_normal(K).astype(np.float32)), dev.upload(np.ones(K, np.float32))
    kc0, vc0 = rng.standard_normal((n_ctx, E)).astype(ct), rng.standard_normal((n_ctx, E)).astype(ct)
    hm = lambda c: np.ascontiguousarray(c.reshape(n_ctx, H, D).transpose(1, 0, 2))
    pos = dev.upload(np.array([n_past], np.int32))
    res = []
    for layout in (0, n_ctx):
        q, k, v = (dev.alloc(E * 4) for _ in range(3))
        items = dev.gemv_items([{"vx": w, "y": x, "dst": d, "ncols": K, "nrows": E, "norm_weight": nw, "norm_eps": 1e-5}
                                for w, d in zip(ws, (q, k, v))])
        kcb, vcb, out = dev.upload(hm(kc0) if layout else kc0), dev.upload(hm(vc0) if layout else vc0), dev.alloc(E * 4)
        dev.qkv_attn_decode(items, kcb, vcb, out, H, D, n_past, pos, 1.0, 10000.0 ** (-2.0 / D), D ** -0.5, kv_f16=kv_f16,
                            head_major_n_ctx=layout)
        shape = (H, n_ctx, D) if layout else (n_ctx, E)
        o, kg, vg = dev.download(out, np.float32, E), dev.download(kcb, ct, shape), dev.download(vcb, ct, shape)
        if layout:
            kg, vg = kg.transpose(1, 0, 2).reshape(n_ctx, E), vg.transpose(1, 0, 2).reshape(n_ctx, E)
        res.append((o, kg, vg))
        for b in (q, k, v, kcb, vcb, out):
            dev.free(b)
    for a, b in zip(*res):
        assert np.array_equal(a.view(np.uint8), b.view(np.uint8))
    assert np.all(np.isfinite(res[1][0]))
    for b in ws + [x, nw, pos]:
        dev.free(b)


def test_qkv_attn_argument_errors(dev):
    from galois_amd import GaloisHipError
    rng = np.random.default_rng(1)
    H, D, K = 2, 128, 256
    E = H * D
    w = dev.upload(oracle.quantize_q4_0((rng.standard_normal((E, K)) * 0.05).astype(np.float32)))
    x, q, kc, out = dev.upload(np.ones(K, np.float32)), dev.alloc(E * 4), dev.alloc(4 * E * 4), dev.alloc(E * 4)
    pos = dev.upload(np.array([0], np.int32))
    item = {"vx": w, "y": x, "dst": q, "ncols": K, "nrows": E}
    ok = [item, item, item]
    for items, h, d, code in ((ok, H, 64, -5),                                           # heads of 128 only
                              ([item, item, dict(item, nrows=E - 16)], H, D, -2),        # every product n_head * head_dim rows
                              ([item, item, dict(item, residual=x)], H, D, -5),          # no residual, pair or second output
                              (ok, 0, D, -2),
                              ([dict(item, ncols=12288)] * 3, H, D, -2)):                # vectors of up to 11776
        with pytest.raises(GaloisHipError) as ei:
            dev.qkv_attn_decode(items, kc, kc, out, h, d, 0, pos, 1.0, 0.9, 0.1)
        assert ei.value.status == code, (ei.value.status, code)
    for b in (w, x, q, kc, out, pos):
        dev.free(b)


def test_qkv_attn_repeated_calls(dev):
    """Counters return to zero: the same launch again and again, and a different head count after it."""
    _case(dev, 32, 4096, 1500, 2, False, seed=5, repeats=6)
    _case(dev, 5, 256, 700, 1, False, seed=6, repeats=3)
    _case(dev, 32, 4096, 100, 1, True, seed=7, repeats=3)


@pytest.mark.parametrize("H,K,n_past", [(32, 4096, 2047), (3, 256, 40)])
def test_a_wait_that_runs_out_is_reported_and_leaves_the_context_usable(dev, H, K, n_past):
    """The give-up path of the waits inside the launch, forced from the host: the attention workgroups wait for one
    count more than the products can reach, with a bound of a few polls, so every wait runs out and every kernel
    still ends normally.  Every head's output is NaN in all its elements, the products themselves are right, the next
    synchronize reports GALOIS_HIP_E_DEVICE_WAIT exactly once, and the same call afterwards -- with the default
    settings -- gives what it gave before, bit for bit (the counters the late products left non-zero are cleared)."""
    from galois_amd import GaloisHipError
    D = 128
    E = H * D
    rng = np.random.default_rng(90 + H)
    ws = [dev.upload(oracle.quantize_q4_0((rng.standard_normal((E, K)) * 0.05).astype(np.float32))) for _ in range(3)]
    x = dev.upload(rng.standard_normal(K).astype(np.float32))
    kc0 = rng.standard_normal((n_past + 1, E)).astype(np.float32)
    vc0 = rng.standard_normal((n_past + 1, E)).astype(np.float32)
    pos = dev.upload(np.array([n_past], np.int32))
    q, k, v, out = (dev.alloc(E * 4) for _ in range(4))
    kc, vc = dev.upload(kc0), dev.upload(vc0)
    items = dev.gemv_items([{"vx": w, "y": x, "dst": d, "ncols": K, "nrows": E} for w, d in zip(ws, (q, k, v))])
    args = (items, kc, vc, out, H, D, n_past, pos, 1.0, 10000.0 ** (-2.0 / D), D ** -0.5)

    def run():
        dev.upload(kc0, kc), dev.upload(vc0, vc)
        dev.qkv_attn_decode(*args)
        dev.synchronize()
        return [dev.download(b, np.float32, E) for b in (q, k, v, out)]

    good = run()
    assert np.all(np.isfinite(good[3]))
    print("give-up case H=%d K=%d n_past=%d" % (H, K, n_past), flush=True)
    dev.set_option(dev.OPT_WAIT_SPIN_LIMIT, 4)
    dev.set_option(dev.OPT_WAIT_TARGET_BIAS, 1)
    try:
        dev.upload(kc0, kc), dev.upload(vc0, vc)
        dev.qkv_attn_decode(*args)
        with pytest.raises(GaloisHipError) as ei:
            dev.synchronize()
        assert ei.value.status == -7
        dev.synchronize()                                   # reported once
        bad = [dev.download(b, np.float32, E) for b in (q, k, v, out)]
        assert np.all(np.isnan(bad[3])), "every element of every head is poisoned"
        for a, b in zip(good[:3], bad[:3]):                 # the products do not depend on the waits
            assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
    finally:
        dev.set_option(dev.OPT_WAIT_TARGET_BIAS, 0)
        dev.set_option(dev.OPT_WAIT_SPIN_LIMIT, 0)
    for _ in range(2):
        again = run()
        for a, b in zip(good, again):
            assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
    for b in ws + [x, pos, q, k, v, out, kc, vc]:
        dev.free(b)
