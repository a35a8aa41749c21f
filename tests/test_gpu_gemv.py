"""GPU parity of the Q4_0 decode GEMV (through the C ABI) against the CPU oracle.

Bar (BASELINE north_star): f32 outputs within 1e-4 relative of the dequant-then-dot oracle,
measured both as max|d|/max|ref| and as relative L2.
"""
import json
import os

import numpy as np
import pytest

import oracle
from tests import npref

pytestmark = pytest.mark.gpu
TOL = 1e-4
KAT = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "kat.json")))


def _gemv(dev, wq, x, x_off_bytes=0, w_off_bytes=0):
    n = wq.shape[0]
    k = x.size
    wbuf = dev.alloc(wq.nbytes + 64)
    xbuf = dev.alloc(x.nbytes + 64)
    ybuf = dev.alloc(n * 4 + 64)
    canary = np.full(n + 16, 7.5, np.float32)
    dev.upload(canary, ybuf)
    dev.upload(wq, wbuf.view(w_off_bytes))
    dev.upload(x, xbuf.view(x_off_bytes))
    dev.dequantize_mul_mat_vec_q4_0(wbuf.view(w_off_bytes), xbuf.view(x_off_bytes), ybuf, k, n)
    out = dev.download(ybuf, np.float32, n + 16)
    assert np.all(out[n:] == 7.5), "wrote past the end of dst"
    for b in (wbuf, xbuf, ybuf):
        dev.free(b)
    return out[:n]


def _case(seed, k, n, wscale=0.02):
    rng = np.random.default_rng(seed)
    w = (rng.standard_normal((n, k)) * wscale).astype(np.float32)
    x = rng.standard_normal(k).astype(np.float32)
    return oracle.quantize_q4_0(w), x


def test_gemv_kat(dev):
    c = KAT["gemv"]
    wq = np.array(c["W"], np.uint8)
    for case in c["cases"]:
        x = np.array(case["x"], np.float32)
        assert _gemv(dev, wq, x).tolist() == case["y"]


@pytest.mark.parametrize("k,n", [(64, 1), (64, 5), (128, 3), (4096, 16), (4096, 17), (4096, 255), (11008, 33),
                                 (12288 + 64, 9), (64 * 200, 4), (256, 4096)])
def test_gemv_fast_path_small(dev, k, n):
    wq, x = _case(k * 31 + n, k, n)
    ref = oracle.mul_mat_q4_0_f32(wq, x)
    got = _gemv(dev, wq, x)
    emax, el2 = npref.rel_err(got, ref)
    assert emax < TOL and el2 < TOL, (k, n, emax, el2)


@pytest.mark.parametrize("k,n", [(32, 1), (32, 7), (96, 5), (4096 + 32, 13)])
def test_gemv_generic_path_odd_block_count(dev, k, n):
    wq, x = _case(k + n, k, n)
    ref = oracle.mul_mat_q4_0_f32(wq, x)
    emax, el2 = npref.rel_err(_gemv(dev, wq, x), ref)
    assert emax < TOL and el2 < TOL


def test_gemv_generic_path_misaligned_pointers(dev):
    wq, x = _case(5, 4096, 21)
    ref = oracle.mul_mat_q4_0_f32(wq, x)
    for woff, xoff in ((2, 0), (0, 4), (18, 8)):
        emax, el2 = npref.rel_err(_gemv(dev, wq, x, x_off_bytes=xoff, w_off_bytes=woff), ref)
        assert emax < TOL and el2 < TOL, (woff, xoff)


@pytest.mark.parametrize("k,n", [(4096, 4096), (4096, 11008), (11008, 4096), (4096, 32000)])
def test_gemv_llama7b_shapes(dev, k, n):
    wq, x = _case(k ^ n, k, n)
    ref = oracle.mul_mat_q4_0_f32(wq, x)
    got = _gemv(dev, wq, x)
    emax, el2 = npref.rel_err(got, ref)
    print("gemv K=%d N=%d max_rel=%.3g l2_rel=%.3g" % (k, n, emax, el2))
    assert emax < TOL and el2 < TOL


def test_gemv_special_values(dev):
    k, n = 4096, 64
    wq, x = _case(77, k, n)
    w = npref.q4_0_dequant(wq)
    # unit vectors select exact columns of the dequantised matrix
    for kk in (0, 15, 16, 31, 32, 63, 64, 4095):
        e = np.zeros(k, np.float32)
        e[kk] = 1.0
        assert np.array_equal(_gemv(dev, wq, e), w[:, kk]), kk
    # all-0x88 blocks are all-zero weights whatever the scale
    z = np.tile(np.array([0x00, 0x3C] + [0x88] * 16, np.uint8), (n, k // 32))
    # (the kernel forms sum(n*x) - 8*sum(x), so "zero" is zero to f32 rounding of those two sums)
    assert np.max(np.abs(_gemv(dev, z, x))) <= 1e-6 * 8.0 * np.sum(np.abs(x))
    # negative / tiny / large scales
    for wscale in (1e-6, 50.0):
        wq2, x2 = _case(78, k, n, wscale)
        emax, el2 = npref.rel_err(_gemv(dev, wq2, x2), oracle.mul_mat_q4_0_f32(wq2, x2))
        assert emax < TOL and el2 < TOL, wscale
    # linearity in x (size-independent property)
    a = _gemv(dev, wq, x)
    b = _gemv(dev, wq, (2 * x).astype(np.float32))
    assert np.allclose(b, 2 * a, rtol=1e-6, atol=1e-6)


def test_gemv_argument_errors(dev):
    from galois_amd import GaloisHipError
    buf = dev.alloc(4096)
    for args, code in (((buf, buf, buf, 48, 1), -2), ((buf, buf, buf, 0, 1), -2), ((buf, buf, buf, 32, 0), -2),
                       ((None, buf, buf, 32, 1), -1), ((buf.view(1), buf, buf, 32, 1), -3),
                       ((buf, buf.view(2), buf, 32, 1), -3)):
        with pytest.raises(GaloisHipError) as ei:
            dev.dequantize_mul_mat_vec_q4_0(*args)
        assert ei.value.status == code
    dev.free(buf)
