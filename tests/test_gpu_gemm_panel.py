"""The prefill matmul on an fp16 panel (activations already in the order the matrix instructions fetch them) and the
ops that write the panel, through the C ABI.

Bars: the panel written by galois_hip_f32_to_f16_panel is the f32 matrix rounded to fp16 (numpy's nearest-even), tile
for tile; a matmul on it equals galois_hip_mul_mat_q4_0_f32 on the f32 matrix bit for bit, alone or as one of several
matrices in a launch; the norm and SwiGLU producers hold fp16(their f32 op) up to one unit in the last place of fp16
(their reductions and exponentials round like the f32 ops', whose results the oracle gives to 1e-6), and the product
on their panels is within the prefill bar (2e-3) of the oracle's f64 dequantize-then-GEMM on the oracle's activations.
"""
import numpy as np
import pytest

import oracle
from tests import npref

pytestmark = pytest.mark.gpu
TOL = 2e-3


def _untile(raw, m, k):
    """Panel bytes -> [m_pad, k] float16: tile (r16, c32) is 1 KB, its 16-byte piece (g, r) holds columns c32*32 + g*8 .."""
    m_pad = (m + 15) // 16 * 16
    t = raw.view(np.float16).reshape(m_pad // 16, k // 32, 4, 16, 8)
    return t.transpose(0, 3, 1, 2, 4).reshape(m_pad, k)


def _panel(dev, k, m):
    n = dev.f16_panel_bytes(k, m)
    assert n == (m + 15) // 16 * 16 * k * 2
    return dev.alloc(n), n


def _case(seed, m, k, ns):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((m, k)).astype(np.float32)
    wqs = [oracle.quantize_q4_0((rng.standard_normal((n, k)) * 0.02).astype(np.float32)) for n in ns]
    return x, wqs


@pytest.mark.parametrize("m,k", [(512, 4096), (130, 256), (1, 512), (17, 11008)])
def test_the_panel_is_the_matrix_rounded_to_fp16(dev, m, k):
    x, _ = _case(m + k, m, k, [])
    xb = dev.upload(x)
    pb, nbytes = _panel(dev, k, m)
    dev.upload(np.full(nbytes // 4, 7.5, np.float32), pb)
    dev.f32_to_f16_panel(xb, pb, k, m)
    got = _untile(dev.download(pb, np.uint8, nbytes), m, k)
    assert np.array_equal(got[:m].view(np.uint16), x.astype(np.float16).view(np.uint16))
    assert np.all(got[m:] == 0), "rows past M are zero"
    for b in (xb, pb):
        dev.free(b)


@pytest.mark.parametrize("m,k,ns", [(512, 4096, [4096, 4096, 4096]), (512, 4096, [11008, 11008]), (512, 4096, [11008]),
                                    (130, 256, [100, 4096, 177, 48]), (300, 1024, [96, 97]), (16, 2048, [5000])])
def test_matmul_on_the_panel_equals_the_f32_call_bit_for_bit(dev, m, k, ns):
    x, wqs = _case(m * 3 + k + len(ns), m, k, ns)
    xb = dev.upload(x)
    wbs = [dev.upload(w) for w in wqs]
    pb, _ = _panel(dev, k, m)
    dev.f32_to_f16_panel(xb, pb, k, m)
    ys = [dev.alloc((m * n + 16) * 4) for n in ns]
    for y, n in zip(ys, ns):
        dev.upload(np.full(m * n + 16, 7.5, np.float32), y)
    print("panel matmul m=%d k=%d ns=%s" % (m, k, ns), flush=True)
    dev.mul_mat_q4_0_f16_panel([(w, y, n) for w, y, n in zip(wbs, ys, ns)], pb, k, m)
    ref = dev.alloc(m * max(ns) * 4)
    for w, wq, y, n in zip(wbs, wqs, ys, ns):
        got = dev.download(y, np.float32, m * n + 16)
        assert np.all(got[m * n:] == 7.5), "wrote past the end of Y"
        dev.mul_mat_q4_0_f32(w, xb, ref, k, n, m)
        one = dev.download(ref, np.float32, m * n)
        assert np.array_equal(got[:m * n].view(np.uint32), one.view(np.uint32)), n
        cols = np.unique(np.concatenate([[0, n - 1], np.random.default_rng(n).choice(n, min(n, 64), replace=False)]))
        emax, el2 = npref.rel_err(got[:m * n].reshape(m, n)[:, cols], oracle.mul_mat_q4_0_f32(wq[cols], x))
        assert emax < TOL and el2 < TOL, (n, emax, el2)
    for b in [xb, pb, ref] + wbs + ys:
        dev.free(b)


@pytest.mark.parametrize("m,k,n", [(512, 4096, 4096), (512, 11008, 4096), (512, 4096, 11008), (130, 256, 200), (300, 768, 1000),
                                   (17, 512, 4096), (600, 2816, 2048)])
@pytest.mark.parametrize("with_residual", [True, False])
def test_matmul_with_the_residual_folded_in_and_in_two_shares_of_k(dev, m, k, n, with_residual):
    """Y = residual + W . panel.  Without a workspace the call is the plain product and a pass that adds the residual:
    bit for bit the plain call's result plus the residual.  With a workspace a narrow matrix runs as two shares
    of k (the first two shapes on 256 CUs) -- another order of the f32 sums, so that result is held to the prefill bar
    against the oracle, and to 1e-5 of the largest magnitude against the one-launch result; Y may be the residual."""
    x, (wq,) = _case(m + k + n, m, k, [n])
    r = np.random.default_rng(n).standard_normal((m, n)).astype(np.float32) if with_residual else None
    xb, wb = dev.upload(x), dev.upload(wq)
    pb, _ = _panel(dev, k, m)
    dev.f32_to_f16_panel(xb, pb, k, m)
    rb = dev.upload(r) if with_residual else None
    plain, one, two = dev.alloc(m * n * 4), dev.alloc((m * n + 16) * 4), dev.alloc((m * n + 16) * 4)
    ws_bytes = 2 * m * n * 4
    ws = dev.alloc(ws_bytes + 64)
    for b in (one, two):
        dev.upload(np.full(m * n + 16, 7.5, np.float32), b)
    dev.upload(np.full(ws_bytes // 4 + 16, 9.5, np.float32), ws)
    dev.mul_mat_q4_0_f16_panel([(wb, plain, n)], pb, k, m)
    dev.mul_mat_q4_0_f16_panel_add(wb, pb, rb, one, k, n, m)
    dev.mul_mat_q4_0_f16_panel_add(wb, pb, rb, two, k, n, m, ws, ws_bytes)
    base = dev.download(plain, np.float32, m * n).reshape(m, n)
    got1, got2 = dev.download(one, np.float32, m * n + 16), dev.download(two, np.float32, m * n + 16)
    assert np.all(got1[m * n:] == 7.5) and np.all(got2[m * n:] == 7.5), "wrote past the end of Y"
    assert np.all(dev.download(ws, np.float32, ws_bytes // 4 + 16)[ws_bytes // 4:] == 9.5), "wrote past the end of the workspace"
    got1, got2 = got1[:m * n].reshape(m, n), got2[:m * n].reshape(m, n)
    want = base + r if with_residual else base
    assert np.array_equal(got1.view(np.uint32), want.view(np.uint32))
    assert np.max(np.abs(got2 - want)) <= 1e-5 * np.max(np.abs(want))
    cols = np.unique(np.concatenate([[0, n - 1], np.random.default_rng(n).choice(n, min(n, 48), replace=False)]))
    ref = oracle.mul_mat_q4_0_f32(wq[cols], x)
    emax, el2 = npref.rel_err(got2[:, cols] - (r[:, cols] if with_residual else 0), ref)
    assert emax < TOL and el2 < TOL, (emax, el2)
    if with_residual:   # in place on the residual stream
        dev.mul_mat_q4_0_f16_panel_add(wb, pb, rb, rb, k, n, m, ws, ws_bytes)
        assert np.array_equal(dev.download(rb, np.float32, m * n).reshape(m, n).view(np.uint32), got2.view(np.uint32))
        from galois_amd import GaloisHipError
        with pytest.raises(GaloisHipError) as ei:      # in place needs somewhere to keep the product
            dev.mul_mat_q4_0_f16_panel_add(wb, pb, rb, rb, k, n, m)
        assert ei.value.status == -5
    for b in [xb, wb, pb, plain, one, two, ws] + ([rb] if with_residual else []):
        dev.free(b)


@pytest.mark.parametrize("m,k,n", [(512, 11008, 4096), (512, 4096, 4096), (130, 256, 512), (33, 768, 2048)])
@pytest.mark.parametrize("with_residual", [True, False])
def test_shares_then_adding_pass_fused_with_the_next_norm(dev, m, k, n, with_residual):
    """The product left as its shares of k, then one launch that adds them (and the residual) and writes the next
    norm's panel: the sum and the panel equal, bit for bit, those of the folded matmul followed by the norm-to-panel
    call (the same additions in the same order, the same norm arithmetic)."""
    x, (wq,) = _case(m + k + n + 1, m, k, [n])
    rng = np.random.default_rng(n + m)
    r = rng.standard_normal((m, n)).astype(np.float32) if with_residual else None
    g = (1 + 0.1 * rng.standard_normal(n)).astype(np.float32)
    xb, wb, gb = dev.upload(x), dev.upload(wq), dev.upload(g)
    rb = dev.upload(r) if with_residual else None
    pb, _ = _panel(dev, k, m)
    dev.f32_to_f16_panel(xb, pb, k, m)
    ws_bytes = 2 * m * n * 4
    ws, y_ref, y_got = dev.alloc(ws_bytes), dev.alloc(m * n * 4), dev.alloc(m * n * 4)
    p_ref, nb = _panel(dev, n, m)
    p_got, _ = _panel(dev, n, m)
    dev.mul_mat_q4_0_f16_panel_add(wb, pb, rb, y_ref, k, n, m, ws, ws_bytes)
    dev.rms_norm_mul_f16_panel(y_ref, gb, p_ref, n, m, 1e-6)
    shares = dev.mul_mat_q4_0_f16_panel_shares(wb, pb, ws, ws_bytes, k, n, m)
    assert shares in (1, 2)
    if m == 512 and dev.info()["n_cu"] == 256:
        assert shares == 2      # 4096 columns at 512 rows leave CUs idle as whole-k tiles
    dev.add_rms_norm_mul_f16_panel(ws, ws.view(m * n * 4) if shares == 2 else None, rb, y_got, gb, p_got, n, m, 1e-6)
    assert np.array_equal(dev.download(y_got, np.uint32, m * n), dev.download(y_ref, np.uint32, m * n))
    assert np.array_equal(dev.download(p_got, np.uint8, nb), dev.download(p_ref, np.uint8, nb))
    # with room for one result only the product comes whole
    assert dev.mul_mat_q4_0_f16_panel_shares(wb, pb, ws, m * n * 4, k, n, m) == 1
    if with_residual:   # the sum may replace the residual in place
        dev.add_rms_norm_mul_f16_panel(ws, None, rb, rb, gb, p_got, n, m, 1e-6)
        whole = dev.download(ws, np.float32, m * n)
        assert np.array_equal(dev.download(rb, np.float32, m * n), whole + r.reshape(-1))
    for b in [xb, wb, gb, pb, ws, y_ref, y_got, p_ref, p_got] + ([rb] if with_residual else []):
        dev.free(b)


@pytest.mark.parametrize("m,k,n", [(512, 4096, 11008), (130, 256, 512), (33, 768, 256), (300, 1024, 2816), (1, 512, 768)])
def test_gate_up_and_swiglu_in_one_launch(dev, m, k, n):
    """The panel of silu(Wg . x) * (Wu . x) from one launch against the panel that the two-matrix matmul followed by
    the SwiGLU-to-panel call writes: the products are the same bits and the SwiGLU the same expression, but the compiler
    is free to fuse 1 + exp(-g) into the exponential's last step in one kernel and not in the other, so a few elements
    (here: fewer than one in a thousand) differ by one unit in the last place of fp16; rows past m are zeros; the down
    projection on the panel meets twice the prefill bar against the oracle's ops on the oracle's activations."""
    x, (wg, wu) = _case(m + k + n + 7, m, k, [n, n])
    rng = np.random.default_rng(k + n)
    n_out = 160
    wd = oracle.quantize_q4_0((rng.standard_normal((n_out, n)) * 0.02).astype(np.float32))
    xb, gb, ub, db = dev.upload(x), dev.upload(wg), dev.upload(wu), dev.upload(wd)
    pb, _ = _panel(dev, k, m)
    dev.f32_to_f16_panel(xb, pb, k, m)
    p_ref, nb = _panel(dev, n, m)
    p_got, _ = _panel(dev, n, m)
    dev.upload(np.full(nb // 4, 7.5, np.float32), p_got)
    yg, yu, yd = dev.alloc(m * n * 4), dev.alloc(m * n * 4), dev.alloc(m * n_out * 4)
    dev.mul_mat_q4_0_f16_panel([(gb, yg, n), (ub, yu, n)], pb, k, m)
    dev.silu_mul_f16_panel(yg, yu, p_ref, n, m)
    dev.mul_mat_q4_0_swiglu_f16_panel(gb, ub, pb, p_got, k, n, m)
    got, ref = _untile(dev.download(p_got, np.uint8, nb), m, n), _untile(dev.download(p_ref, np.uint8, nb), m, n)
    assert _ulps_f16(got[:m], ref[:m]) <= 1.0
    assert np.count_nonzero(got[:m] != ref[:m]) <= max(1, got[:m].size // 1000)
    assert np.all(got[m:] == 0)
    dev.mul_mat_q4_0_f16_panel([(db, yd, n_out)], p_got, n, m)
    act = oracle.mul(oracle.silu(oracle.mul_mat_q4_0_f32(wg, x)).reshape(-1), oracle.mul_mat_q4_0_f32(wu, x).reshape(-1)).reshape(m, n)
    emax, el2 = npref.rel_err(dev.download(yd, np.float32, (m, n_out)), oracle.mul_mat_q4_0_f32(wd, act))
    assert emax < 2 * TOL and el2 < 2 * TOL, (emax, el2)      # two products and a rounding to fp16 in a row
    for b in (xb, gb, ub, db, pb, p_ref, p_got, yg, yu, yd):
        dev.free(b)


def _ulps_f16(a, b):
    """Largest distance between two float16 arrays in units of the last place of the larger magnitude."""
    a32, b32 = a.astype(np.float32), b.astype(np.float32)
    ulp = np.maximum(np.spacing(np.maximum(np.abs(a), np.abs(b)).astype(np.float16)).astype(np.float32), 2.0 ** -24)
    return float(np.max(np.abs(a32 - b32) / ulp))


@pytest.mark.parametrize("m,k,n", [(512, 4096, 4096), (130, 256, 200), (33, 11008, 96), (5, 16384, 64)])
def test_rms_norm_into_the_panel(dev, m, k, n):
    rng = np.random.default_rng(m + k)
    x = (rng.standard_normal((m, k)) * rng.uniform(0.1, 4.0, (m, 1))).astype(np.float32)
    g = (1 + 0.1 * rng.standard_normal(k)).astype(np.float32)
    wq = oracle.quantize_q4_0((rng.standard_normal((n, k)) * 0.02).astype(np.float32))
    xb, gb, wb, yb = dev.upload(x), dev.upload(g), dev.upload(wq), dev.alloc(m * n * 4)
    pb, nbytes = _panel(dev, k, m)
    dev.upload(np.full(nbytes // 4, 7.5, np.float32), pb)
    dev.rms_norm_mul_f16_panel(xb, gb, pb, k, m, 1e-6)
    act = oracle.mul(oracle.rms_norm(x, 1e-6), g)
    got = _untile(dev.download(pb, np.uint8, nbytes), m, k)
    assert np.all(got[m:] == 0)
    assert _ulps_f16(got[:m], act.astype(np.float16)) <= 1.0
    dev.mul_mat_q4_0_f16_panel([(wb, yb, n)], pb, k, m)
    emax, el2 = npref.rel_err(dev.download(yb, np.float32, (m, n)), oracle.mul_mat_q4_0_f32(wq, act))
    assert emax < TOL and el2 < TOL, (emax, el2)
    for b in (xb, gb, wb, yb, pb):
        dev.free(b)


@pytest.mark.parametrize("m,k,n", [(512, 11008, 512), (130, 256, 200), (1, 768, 33)])
def test_swiglu_into_the_panel(dev, m, k, n):
    rng = np.random.default_rng(m * 5 + k)
    gate = (rng.standard_normal((m, k)) * 2).astype(np.float32)
    up = rng.standard_normal((m, k)).astype(np.float32)
    wq = oracle.quantize_q4_0((rng.standard_normal((n, k)) * 0.02).astype(np.float32))
    gb, ub, wb, yb = dev.upload(gate), dev.upload(up), dev.upload(wq), dev.alloc(m * n * 4)
    pb, nbytes = _panel(dev, k, m)
    dev.silu_mul_f16_panel(gb, ub, pb, k, m)
    act = oracle.mul(oracle.silu(gate).reshape(-1), up.reshape(-1)).reshape(m, k)
    got = _untile(dev.download(pb, np.uint8, nbytes), m, k)
    assert np.all(got[m:] == 0)
    assert _ulps_f16(got[:m], act.astype(np.float16)) <= 1.0
    dev.mul_mat_q4_0_f16_panel([(wb, yb, n)], pb, k, m)
    emax, el2 = npref.rel_err(dev.download(yb, np.float32, (m, n)), oracle.mul_mat_q4_0_f32(wq, act))
    assert emax < TOL and el2 < TOL, (emax, el2)
    for b in (gb, ub, wb, yb, pb):
        dev.free(b)


def test_panel_argument_errors(dev):
    from galois_amd import GaloisHipError
    buf = dev.alloc(1 << 16)
    with pytest.raises(GaloisHipError) as ei:
        dev.f16_panel_bytes(100, 4)                        # K must be a multiple of 256
    assert ei.value.status == -2
    for call, code in ((lambda: dev.f32_to_f16_panel(buf, buf, 128, 4), -2),
                       (lambda: dev.f32_to_f16_panel(buf.view(4), buf, 256, 4), -3),
                       (lambda: dev.rms_norm_mul_f16_panel(buf, None, buf, 256, 4, 1e-6), -1),
                       (lambda: dev.silu_mul_f16_panel(buf, buf, buf, 256, 0), -2),
                       (lambda: dev.mul_mat_q4_0_f16_panel([], buf, 256, 4), -2),
                       (lambda: dev.mul_mat_q4_0_f16_panel([(buf, buf, 8)] * 5, buf, 256, 4), -2),
                       (lambda: dev.mul_mat_q4_0_f16_panel([(buf.view(2), buf, 8)], buf, 256, 4), -3),
                       (lambda: dev.mul_mat_q4_0_f16_panel([(buf, buf, 0)], buf, 256, 4), -2)):
        with pytest.raises(GaloisHipError) as ei:
            call()
        assert ei.value.status == code, (ei.value.status, code)
    dev.free(buf)
