"""GPU parity of the row kernels (RMSNorm, RoPE, softmax) through the C ABI vs the CPU oracle."""
import json
import os

import numpy as np
import pytest

import oracle
from tests import npref

pytestmark = pytest.mark.gpu
KAT = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "kat.json")))


def _run(dev, fn, x, *args, extra=()):
    """Uploads x (+ extra arrays), runs fn(xbuf, ybuf-with-canary, ...), returns y like x."""
    xbuf = dev.upload(x)
    ebufs = [dev.upload(e) for e in extra]
    ybuf = dev.alloc(x.nbytes + 256)
    dev.upload(np.full(x.size + 64, 7.5, np.float32), ybuf)
    fn(xbuf, ybuf, ebufs, *args)
    out = dev.download(ybuf, np.float32, x.size + 64)
    assert np.all(out[x.size:] == 7.5), "wrote past the end of dst"
    for b in [xbuf, ybuf] + ebufs:
        dev.free(b)
    return out[:x.size].reshape(x.shape)


# ------------------------------------------------------------------ RMSNorm
def _rms(dev, x, eps, w=None):
    nrows, ncols = x.shape
    if w is None:
        return _run(dev, lambda xb, yb, eb: dev.rms_norm_f32(xb, yb, ncols, nrows, eps), x)
    return _run(dev, lambda xb, yb, eb: dev.rms_norm_mul_f32(xb, eb[0], yb, ncols, nrows, eps), x, extra=[w])


def test_rms_norm_kat(dev):
    c = KAT["rms_norm"]
    got = _rms(dev, np.array(c["x"], np.float32), c["eps"])
    assert np.allclose(got, np.array(c["y"]), rtol=2e-6, atol=0)


@pytest.mark.parametrize("nrows,ncols", [(1, 4), (3, 32), (5, 1000), (7, 1021), (4, 4096), (2, 8192), (2, 16384),
                                         (2, 20000), (512, 4096)])
def test_rms_norm_vs_oracle(dev, nrows, ncols):
    rng = np.random.default_rng(nrows + ncols)
    x = rng.standard_normal((nrows, ncols)).astype(np.float32)
    w = (1 + 0.1 * rng.standard_normal(ncols)).astype(np.float32)
    emax, el2 = npref.rel_err(_rms(dev, x, 1e-6), oracle.rms_norm(x, 1e-6))
    assert emax < 1e-5 and el2 < 1e-5
    emax, el2 = npref.rel_err(_rms(dev, x, 1e-6, w), oracle.mul(oracle.rms_norm(x, 1e-6), w))
    assert emax < 1e-5 and el2 < 1e-5


# ------------------------------------------------------------------ RoPE
def _rope(dev, x, pos, freq_scale, p_delta_rows, theta_scale):
    nrows, ncols = x.shape
    return _run(dev, lambda xb, yb, eb: dev.rope_f32(xb, yb, ncols, nrows, eb[0], freq_scale, p_delta_rows,
                                                     theta_scale), x, extra=[np.asarray(pos, np.int32)])


def test_rope_kat(dev):
    c = KAT["rope"]
    x = np.array(c["x"], np.float32)
    got = _rope(dev, x, c["pos"], c["freq_scale"], c["p_delta_rows"], c["theta_scale"])
    assert np.allclose(got, np.array(c["y"]), rtol=0, atol=1e-6)
    assert np.array_equal(got[0], x[0])


@pytest.mark.parametrize("t,h,hd,p0", [(1, 1, 2, 0), (3, 5, 64, 100), (9, 32, 128, 2040), (512, 32, 128, 0),
                                       (4, 7, 258, 17)])
def test_rope_vs_oracle(dev, t, h, hd, p0):
    rng = np.random.default_rng(t + h + hd)
    x = rng.standard_normal((t * h, hd)).astype(np.float32)
    pos = np.arange(p0, p0 + t, dtype=np.int32)
    ts = float(np.float32(10000.0) ** np.float32(-2.0 / hd))
    got = _rope(dev, x, pos, 1.0, h, ts)
    # The gate: the reference kernel's own f32 angle (rope.cu:16-20), rotation in f64.  What separates an f32 kernel
    # from it is an ulp of powf times the angle (~1e-4 rad at position 2000) and f32 sin / cos: 3e-4 absolute on
    # N(0,1) data.  A wrong exponent, pair index or position shows up at 1e-2 and more.
    ref32 = npref.rope_f32_angles(x, pos, 1.0, h, ts)
    err32 = np.max(np.abs(got.astype(np.float64) - ref32))
    assert err32 < 3e-4, err32
    # For information: against the oracle's f64 angle the rounding of the f32 angle itself (6e-8 relative of up to
    # 2500 rad) is included as well.
    ref = oracle.rope(x, pos, 1.0, h, ts)
    err = np.max(np.abs(got.astype(np.float64) - ref))
    print("rope t=%d max abs err vs f32-angle reference %.3g, vs f64-angle oracle %.3g" % (t, err32, err))
    assert err < 2e-3 * max(1.0, (p0 + t) / 512.0)
    # pair norms are preserved to f32 rounding
    n0 = x[:, 0::2].astype(np.float64) ** 2 + x[:, 1::2].astype(np.float64) ** 2
    n1 = got[:, 0::2].astype(np.float64) ** 2 + got[:, 1::2].astype(np.float64) ** 2
    assert np.allclose(n0, n1, rtol=1e-5, atol=1e-6)
    # position 0 is the identity
    got0 = _rope(dev, x, np.zeros(t, np.int32), 1.0, h, ts)
    assert np.array_equal(got0, x)


@pytest.mark.parametrize("kv_f16", [False, True])
@pytest.mark.parametrize("with_v", [False, True])
@pytest.mark.parametrize("t,h,hd,p0", [(1, 1, 4, 0), (3, 5, 64, 100), (77, 32, 128, 1971), (512, 32, 128, 0), (4, 7, 256, 17), (9, 3, 36, 5)])
def test_rope_of_q_and_k_with_the_append_in_one_launch(dev, t, h, hd, p0, with_v, kv_f16):
    """galois_hip_rope_qk_append against the calls it replaces: q_out and the rotated k are galois_hip_rope_f32's bits
    (rope_f32 itself is held to the oracle above); into an f16 cache k and v arrive as numpy's round-to-nearest-even of
    those f32 values; nothing is written past the rows of the call."""
    rng = np.random.default_rng(t + h + hd + p0)
    e = h * hd
    q, k, v = (rng.standard_normal((t * h, hd)).astype(np.float32) for _ in range(3))
    pos = np.arange(p0, p0 + t, dtype=np.int32)
    ts = float(np.float32(10000.0) ** np.float32(-2.0 / hd))
    want_q, want_k = _rope(dev, q, pos, 1.0, h, ts), _rope(dev, k, pos, 1.0, h, ts)
    ct = np.float16 if kv_f16 else np.float32
    qb, kb, vb, pb = dev.upload(q), dev.upload(k), dev.upload(v), dev.upload(pos)
    qo = dev.upload(np.full(t * e + 8, 7.5, np.float32))
    kd, vd = dev.upload(np.full(t * e + 8, 7.5, ct)), dev.upload(np.full(t * e + 8, 7.5, ct))
    dev.rope_qk_append(qb, kb, vb if with_v else None, qo, kd, vd if with_v else None, kv_f16, hd, h, t, pb, 1.0, ts)
    got_q = dev.download(qo, np.float32, t * e + 8)
    got_k, got_v = dev.download(kd, ct, t * e + 8), dev.download(vd, ct, t * e + 8)
    assert np.array_equal(got_q[:t * e].view(np.uint32), want_q.reshape(-1).view(np.uint32))
    assert np.array_equal(got_k[:t * e], want_k.reshape(-1).astype(ct))
    assert np.array_equal(got_v[:t * e], v.reshape(-1).astype(ct) if with_v else np.full(t * e, 7.5, ct))
    for tail in (got_q[t * e:], got_k[t * e:], got_v[t * e:]):
        assert np.all(tail == 7.5)
    for b in (qb, kb, vb, pb, qo, kd, vd):
        dev.free(b)


# ------------------------------------------------------------------ softmax
def _soft(dev, x, causal=None):
    nrows, ncols = x.shape
    if causal is None:
        return _run(dev, lambda xb, yb, eb: dev.soft_max_f32(xb, yb, ncols, nrows), x)
    rph, n_past = causal
    return _run(dev, lambda xb, yb, eb: dev.soft_max_causal_f32(xb, yb, ncols, rph, nrows, n_past), x)


def test_soft_max_kat(dev):
    c = KAT["soft_max"]
    x = np.array([[float(v) for v in c["x"]]], np.float32)
    got = _soft(dev, x)[0]
    assert np.allclose(got, np.array(c["y"]), rtol=1e-6, atol=0)
    assert got[2] == 0.0


@pytest.mark.parametrize("nrows,ncols", [(1, 1), (3, 4), (5, 33), (9, 512), (4, 2048), (3, 4096), (2, 5000),
                                         (2, 8192), (1024, 512)])
def test_soft_max_vs_oracle(dev, nrows, ncols):
    rng = np.random.default_rng(nrows * 3 + ncols)
    x = (rng.standard_normal((nrows, ncols)) * 3).astype(np.float32)
    x[rng.random(x.shape) < 0.1] = -np.inf
    x[:, 0] = 0.0  # no all-masked rows
    got = _soft(dev, x)
    ref = oracle.soft_max(x)
    emax, el2 = npref.rel_err(got, ref)
    assert emax < 1e-5 and el2 < 1e-5
    assert np.all(got[np.isinf(x)] == 0)
    assert np.allclose(got.sum(-1), 1, atol=1e-5)


@pytest.mark.parametrize("heads,rph,ncols,n_past", [(2, 8, 8, 0), (3, 5, 12, 7), (32, 512, 512, 0), (2, 3, 2048, 2045)])
def test_soft_max_causal_vs_oracle(dev, heads, rph, ncols, n_past):
    rng = np.random.default_rng(heads + rph + ncols)
    x = (rng.standard_normal((heads * rph, ncols)) * 3).astype(np.float32)
    got = _soft(dev, x, (rph, n_past))
    ref = oracle.soft_max_causal(x, rph, n_past)
    emax, el2 = npref.rel_err(got, ref)
    assert emax < 1e-5 and el2 < 1e-5
    # masked columns are exactly zero and equal to feeding -inf through the plain kernel
    xm = x.copy()
    for r in range(x.shape[0]):
        xm[r, n_past + (r % rph) + 1:] = -np.inf
    assert np.array_equal(got, _soft(dev, xm))
    if n_past == 0:
        assert np.all(got[::rph, 0] == 1.0)


def test_rowop_argument_errors(dev):
    from galois_amd import GaloisHipError
    buf = dev.alloc(4096)
    with pytest.raises(GaloisHipError) as ei:
        dev.rms_norm_f32(buf, buf, 0, 1, 1e-6)
    assert ei.value.status == -2
    with pytest.raises(GaloisHipError) as ei:
        dev.rope_f32(buf, buf, 3, 1, buf, 1.0, 1, 0.5)
    assert ei.value.status == -2
    with pytest.raises(GaloisHipError) as ei:
        dev.soft_max_f32(None, buf, 4, 1)
    assert ei.value.status == -1
    with pytest.raises(GaloisHipError) as ei:
        dev.soft_max_causal_f32(buf, buf, 4, 0, 1, 0)
    assert ei.value.status == -2
    dev.free(buf)
