"""GPU parity of the grouped decode GEMV (several products per launch, with the RMSNorm, SwiGLU and
residual fusions) against the CPU oracle, through the C ABI.

Bar (BASELINE north_star): f32 outputs within 1e-4 relative of the oracle composed of the same ops
in f64: rms_norm -> mul -> dequant-then-dot -> silu * up -> + residual.
"""
import numpy as np
import pytest

import oracle
from galois_amd import GaloisHipError
from tests import npref

pytestmark = pytest.mark.gpu
TOL = 1e-4


def _wx(seed, k, n, wscale=0.02):
    rng = np.random.default_rng(seed)
    w = (rng.standard_normal((n, k)) * wscale).astype(np.float32)
    return oracle.quantize_q4_0(w)


def _ref_item(it):
    """f64 composition of the oracle's ops for one item (host arrays)."""
    x = it["y"].astype(np.float64)
    if it.get("norm_weight") is not None:
        x = x / np.sqrt(np.mean(x * x) + it["norm_eps"]) * it["norm_weight"].astype(np.float64)
    out = npref.q4_0_dequant(it["vx"]).astype(np.float64) @ x
    if it.get("vx_up") is not None:
        up = npref.q4_0_dequant(it["vx_up"]).astype(np.float64) @ x
        out = out / (1.0 + np.exp(-out)) * up
    if it.get("residual") is not None:
        out = out + it["residual"].astype(np.float64)
    return out


def _run_group(dev, items, in_place_residual=False):
    """Uploads every host array of `items`, runs one grouped launch, returns the outputs."""
    bufs, dev_items, outs = [], [], []
    cache = {}

    def up(a):
        if a is None:
            return None
        if id(a) not in cache:       # the same host array -> the same device vector (shared activations)
            cache[id(a)] = dev.upload(a)
            bufs.append(cache[id(a)])
        return cache[id(a)]

    for it in items:
        n = it["vx"].shape[0]
        dst = dev.alloc(n * 4 + 64)
        bufs.append(dst)
        canary = np.full(n + 16, 7.5, np.float32)
        if in_place_residual and it.get("residual") is not None:
            canary[:n] = it["residual"]
        dev.upload(canary, dst)
        d = {"vx": up(it["vx"]), "y": up(it["y"]), "dst": dst, "ncols": it["y"].size, "nrows": n,
             "vx_up": up(it.get("vx_up")), "norm_weight": up(it.get("norm_weight")),
             "norm_eps": it.get("norm_eps", 0.0),
             "residual": dst if (in_place_residual and it.get("residual") is not None) else up(it.get("residual"))}
        dev_items.append(d)
        outs.append((dst, n))
    dev.dequantize_mul_mat_vec_q4_0_group(dev_items)
    res = []
    for dst, n in outs:
        o = dev.download(dst, np.float32, n + 16)
        assert np.all(o[n:] == 7.5), "wrote past the end of dst"
        res.append(o[:n])
    for b in bufs:
        dev.free(b)
    return res


def _check(got, ref, what):
    emax, el2 = npref.rel_err(got, ref)
    assert emax < TOL and el2 < TOL, (what, emax, el2)


@pytest.mark.parametrize("k,n", [(64, 1), (64, 5), (128, 3), (4096, 16), (4096, 17), (4096, 255), (4096, 4096),
                                 (4160, 9), (11008, 33), (11008, 4096), (12288, 7), (256, 5000)])
def test_group_of_one_matches_oracle_and_single_entry(dev, k, n):
    rng = np.random.default_rng(k * 7 + n)
    wq, x = _wx(k + n, k, n), rng.standard_normal(k).astype(np.float32)
    got, = _run_group(dev, [{"vx": wq, "y": x}])
    _check(got, oracle.mul_mat_q4_0_f32(wq, x), (k, n))
    # same arithmetic as the one-product entry point: per-lane sums and the wave reduction are in the same order
    wb, xb, yb = dev.upload(wq), dev.upload(x), dev.alloc(n * 4)
    dev.dequantize_mul_mat_vec_q4_0(wb, xb, yb, k, n)
    single = dev.download(yb, np.float32, n)
    for b in (wb, xb, yb):
        dev.free(b)
    assert np.array_equal(got, single)


def test_group_llama7b_set_in_one_launch(dev):
    rng = np.random.default_rng(11)
    items = []
    for k, n in [(4096, 4096), (4096, 11008), (11008, 4096), (4096, 32000)]:
        items.append({"vx": _wx(k ^ n, k, n), "y": rng.standard_normal(k).astype(np.float32)})
    for it, got in zip(items, _run_group(dev, items)):
        _check(got, oracle.mul_mat_q4_0_f32(it["vx"], it["y"]), it["vx"].shape)


@pytest.mark.parametrize("k,n", [(4160, 4200), (8192, 4100), (11008, 4113), (12288, 4096), (4224, 9000)])
def test_group_long_vectors_with_many_rows_in_chunks(dev, k, n):
    """More than 16 rows per CU and a vector longer than 4096: the workgroups take the vector in chunks of 64 slots
    (one slot in the last chunk, whole chunks, a ragged one).  Against the oracle, and bit-equal to the one-product
    entry point; beside a short-vector product in the same launch; with activations whose blocks need correction
    planes in every chunk."""
    rng = np.random.default_rng(k + n)
    wq = _wx(k * 3 + n, k, n)
    x = rng.standard_normal(k).astype(np.float32)
    xh = x.copy()
    xh[::32] *= np.float32(2.0 ** 18)        # one outlier per block: every block of every chunk is flagged
    w2, x2 = _wx(5, 4096, 64), rng.standard_normal(4096).astype(np.float32)
    got, got2, goth = _run_group(dev, [{"vx": wq, "y": x}, {"vx": w2, "y": x2}, {"vx": wq, "y": xh}])
    _check(got, oracle.mul_mat_q4_0_f32(wq, x), (k, n))
    _check(got2, oracle.mul_mat_q4_0_f32(w2, x2), "short")
    _check(goth, oracle.mul_mat_q4_0_f32(wq, xh), "outliers")
    wb, xb, yb = dev.upload(wq), dev.upload(x), dev.alloc(n * 4)
    dev.dequantize_mul_mat_vec_q4_0(wb, xb, yb, k, n)
    single = dev.download(yb, np.float32, n)
    for b in (wb, xb, yb):
        dev.free(b)
    assert np.array_equal(got, single)


def test_group_shared_activations_and_ragged_row_counts(dev):
    rng = np.random.default_rng(12)
    x = rng.standard_normal(4096).astype(np.float32)
    x2 = rng.standard_normal(128).astype(np.float32)
    items = [{"vx": _wx(1, 4096, 4096), "y": x}, {"vx": _wx(2, 4096, 1), "y": x}, {"vx": _wx(3, 4096, 77), "y": x},
             {"vx": _wx(4, 128, 4099), "y": x2}, {"vx": _wx(5, 4096, 2), "y": x}, {"vx": _wx(6, 128, 3), "y": x2},
             {"vx": _wx(7, 4096, 513), "y": x}, {"vx": _wx(8, 4096, 64), "y": x}]
    for i, (it, got) in enumerate(zip(items, _run_group(dev, items))):
        _check(got, oracle.mul_mat_q4_0_f32(it["vx"], it["y"]), i)


@pytest.mark.parametrize("k,n", [(4096, 4096), (4096, 130), (11008, 100), (64, 3)])
def test_group_rms_norm_prologue(dev, k, n):
    rng = np.random.default_rng(k + n)
    x = (rng.standard_normal(k) * 3.0).astype(np.float32)
    nw = (1.0 + 0.1 * rng.standard_normal(k)).astype(np.float32)
    it = {"vx": _wx(k * n, k, n), "y": x, "norm_weight": nw, "norm_eps": 1e-6}
    it2 = dict(it, vx=_wx(k * n + 1, k, max(1, n // 2)))   # a second product on the same normalised vector
    plain = {"vx": it["vx"], "y": x}
    (got, got2), (got_plain,) = _run_group(dev, [it, it2]), _run_group(dev, [plain])
    _check(got2, _ref_item(it2), "normed, second matrix")
    _check(got, _ref_item(it), "normed")
    _check(got_plain, _ref_item(plain), "plain")
    # the oracle's own rms_norm and mul agree with the closed form used above
    xn = oracle.mul(oracle.rms_norm(x[None, :], 1e-6), nw)[0]
    _check(got, oracle.mul_mat_q4_0_f32(it["vx"], xn), "normed, oracle ops")


@pytest.mark.parametrize("k,n", [(4096, 11008), (4096, 3), (11008, 65), (64, 1)])
def test_group_swiglu_pair_and_residual(dev, k, n):
    rng = np.random.default_rng(k * 3 + n)
    x = rng.standard_normal(k).astype(np.float32)
    res = rng.standard_normal(n).astype(np.float32)
    it = {"vx": _wx(1 + k, k, n, 0.05), "vx_up": _wx(2 + k, k, n), "y": x}
    it_res = {"vx": _wx(3 + k, k, n), "y": x, "residual": res}
    both = {"vx": it["vx"], "vx_up": it["vx_up"], "y": x, "residual": res,
            "norm_weight": (1.0 + 0.1 * rng.standard_normal(k)).astype(np.float32), "norm_eps": 1e-5}
    a, b = _run_group(dev, [it, it_res])
    _check(a, _ref_item(it), "swiglu")
    _check(b, _ref_item(it_res), "residual")
    c, = _run_group(dev, [both])
    _check(c, _ref_item(both), "norm + swiglu + residual")
    d, = _run_group(dev, [it_res], in_place_residual=True)     # residual aliasing dst: x += W h
    assert np.array_equal(d, b)
    # silu * up composed from the oracle's own silu and mul
    g = oracle.mul_mat_q4_0_f32(it["vx"], x)
    u = oracle.mul_mat_q4_0_f32(it["vx_up"], x)
    _check(a, oracle.silu(g).astype(np.float64) * u, "swiglu, oracle ops")


def test_group_of_six_with_norm_pairs_and_residuals(dev):
    """More than four products per launch take the kernel build that selects among eight argument sets."""
    rng = np.random.default_rng(15)
    x = rng.standard_normal(256).astype(np.float32)
    g = (1 + 0.1 * rng.standard_normal(256)).astype(np.float32)
    items = []
    for i, n in enumerate([33, 1, 700, 64, 129, 16]):
        it = {"vx": _wx(100 + i, 256, n), "y": x, "norm_weight": g, "norm_eps": 1e-5}
        if i % 2 == 0:
            it["vx_up"] = _wx(200 + i, 256, n)
        if i % 3 == 0:
            it["residual"] = rng.standard_normal(n).astype(np.float32)
        items.append(it)
    for i, (it, got) in enumerate(zip(items, _run_group(dev, items))):
        _check(got, _ref_item(it), i)


@pytest.mark.parametrize("k,n1,n2", [(4096, 4096, 11008), (256, 100, 33), (11008, 4096, 300), (64, 17, 5),
                                     # long vectors with many rows (worked in chunks): the producer, then the consumers
                                     (4160, 4224, 300), (4096, 4160, 4200), (11008, 8192, 2100)])
def test_group_norm_split_over_two_launches(dev, k, n1, n2):
    """A launch that produces a vector also writes it times the next norm's weight and its sums of squares per 16
    rows; the next launch consumes those instead of normalising: same result as normalising in the second launch."""
    rng = np.random.default_rng(k + n1)
    h = rng.standard_normal(k).astype(np.float32)
    res = rng.standard_normal(n1).astype(np.float32)
    g = (1 + 0.1 * rng.standard_normal(n1)).astype(np.float32)
    w1, w2, w2u = _wx(1, k, n1), _wx(2, n1, n2) if n1 % 64 == 0 else None, None
    eps = 1e-5
    b = {name: dev.upload(a) for name, a in (("h", h), ("res", res), ("g", g), ("w1", w1))}
    x, xs, sq = dev.alloc(n1 * 4), dev.alloc(n1 * 4), dev.alloc(((n1 + 15) // 16) * 4 + 64)
    dev.upload(np.full((n1 + 15) // 16 + 16, 7.5, np.float32), sq)
    dev.dequantize_mul_mat_vec_q4_0_group([{"vx": b["w1"], "y": b["h"], "dst": x, "ncols": k, "nrows": n1,
                                            "residual": b["res"], "dst_scaled": xs, "scale_weight": b["g"],
                                            "sumsq_out": sq}])
    x_ref = _ref_item({"vx": w1, "y": h, "residual": res})
    x_g = dev.download(x, np.float32, n1)
    _check(x_g, x_ref, "x")
    np.testing.assert_array_equal(dev.download(xs, np.float32, n1), x_g * g)        # one f32 product per element
    sq_g = dev.download(sq, np.float32, (n1 + 15) // 16 + 16)
    assert np.all(sq_g[(n1 + 15) // 16:] == 7.5), "wrote past the end of sumsq_out"
    pad = np.zeros(((n1 + 15) // 16) * 16)
    pad[:n1] = x_g.astype(np.float64) ** 2
    np.testing.assert_allclose(sq_g[:(n1 + 15) // 16], pad.reshape(-1, 16).sum(1), rtol=1e-5)
    if w2 is not None:   # the consuming launch, plain and as a SwiGLU pair, against normalising there
        w2u = _wx(3, n1, n2)
        bw2, bw2u = dev.upload(w2), dev.upload(w2u)
        y_split, y_norm, p_split = dev.alloc(n2 * 4), dev.alloc(n2 * 4), dev.alloc(n2 * 4)
        dev.dequantize_mul_mat_vec_q4_0_group([{"vx": bw2, "y": xs, "dst": y_split, "ncols": n1, "nrows": n2,
                                                "sumsq_in": sq, "norm_eps": eps},
                                               {"vx": bw2, "vx_up": bw2u, "y": xs, "dst": p_split, "ncols": n1,
                                                "nrows": n2, "sumsq_in": sq, "norm_eps": eps}])
        dev.dequantize_mul_mat_vec_q4_0_group([{"vx": bw2, "y": x, "dst": y_norm, "ncols": n1, "nrows": n2,
                                                "norm_weight": b["g"], "norm_eps": eps}])
        ref = _ref_item({"vx": w2, "y": x_g, "norm_weight": g, "norm_eps": eps})
        _check(dev.download(y_split, np.float32, n2), ref, "split")
        _check(dev.download(y_norm, np.float32, n2), ref, "norm")
        _check(dev.download(p_split, np.float32, n2), _ref_item({"vx": w2, "vx_up": w2u, "y": x_g, "norm_weight": g,
                                                                 "norm_eps": eps}), "split pair")
        for t in (bw2, bw2u, y_split, y_norm, p_split):
            dev.free(t)
    for t in list(b.values()) + [x, xs, sq]:
        dev.free(t)


def test_group_special_values(dev):
    k, n = 4096, 40
    wq = _wx(99, k, n)
    w = npref.q4_0_dequant(wq)
    for kk in (0, 17, 63, 4095):       # unit activations select exact columns, whatever shares the launch
        e = np.zeros(k, np.float32)
        e[kk] = 1.0
        got, other = _run_group(dev, [{"vx": wq, "y": e}, {"vx": wq, "y": np.ones(k, np.float32)}])
        assert np.array_equal(got, w[:, kk])
        _check(other, w.astype(np.float64).sum(axis=1), "row sums")


def test_group_split_norm_argument_errors(dev):
    w, x, d = dev.upload(_wx(9, 64, 16)), dev.upload(np.ones(64, np.float32)), dev.alloc(64)
    base = {"vx": w, "y": x, "dst": d, "ncols": 64, "nrows": 16}
    for bad in ({"dst_scaled": d}, {"scale_weight": x}, {"sumsq_out": d, "norm_weight": x},
                {"sumsq_out": d, "vx_up": w}, {"sumsq_in": x, "norm_weight": x, "norm_eps": 1e-5},
                {"dst_scaled": d, "scale_weight": x, "sumsq_in": x}):
        with pytest.raises(GaloisHipError):
            dev.dequantize_mul_mat_vec_q4_0_group([dict(base, **bad)])
    with pytest.raises(GaloisHipError):   # modes may not be mixed in one call
        dev.dequantize_mul_mat_vec_q4_0_group([dict(base, sumsq_in=x, norm_eps=1e-5), dict(base)])
    for t in (w, x, d):
        dev.free(t)


def test_group_argument_errors(dev):
    buf = dev.alloc(1 << 16)
    ok = {"vx": buf, "y": buf, "dst": buf, "ncols": 64, "nrows": 1}
    for items, code in (([], -2), ([ok] * 9, -2), ([dict(ok, ncols=32)], -2), ([dict(ok, nrows=0)], -2),
                        ([dict(ok, vx=None)], -1), ([dict(ok, y=buf.view(4))], -3), ([dict(ok, vx=buf.view(2))], -3),
                        ([dict(ok, ncols=12288 + 64)], -2),
                        ([ok, dict(ok, norm_weight=buf)], -5)):
        with pytest.raises(GaloisHipError) as ei:
            dev.dequantize_mul_mat_vec_q4_0_group(items)
        assert ei.value.status == code, (items, ei.value.status)
    dev.free(buf)
