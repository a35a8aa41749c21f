"""GPU parity of the Q4_0 prefill matmul (MFMA, through the C ABI) against the CPU oracle.

Bar (BASELINE north_star): within 2e-3 relative of dequant-then-GEMM, as max|d|/max|ref|
and as relative L2.
"""
import numpy as np
import pytest

import oracle
from tests import npref

pytestmark = pytest.mark.gpu
TOL = 2e-3


def _gemm(dev, wq, x):
    m, k = x.shape
    n = wq.shape[0]
    wbuf, xbuf = dev.upload(wq), dev.upload(x)
    ybuf = dev.alloc((m * n + 64) * 4)
    dev.upload(np.full(m * n + 64, 7.5, np.float32), ybuf)
    dev.mul_mat_q4_0_f32(wbuf, xbuf, ybuf, k, n, m)
    out = dev.download(ybuf, np.float32, m * n + 64)
    assert np.all(out[m * n:] == 7.5), "wrote past the end of Y"
    for b in (wbuf, xbuf, ybuf):
        dev.free(b)
    return out[:m * n].reshape(m, n)


def _case(seed, m, k, n):
    rng = np.random.default_rng(seed)
    w = (rng.standard_normal((n, k)) * 0.02).astype(np.float32)
    x = rng.standard_normal((m, k)).astype(np.float32)
    return oracle.quantize_q4_0(w), x


@pytest.mark.parametrize("k,n,m", [(64, 160, 130), (256, 200, 130), (1024, 353, 257)])
def test_gemm_layout_probe(dev, k, n, m):
    """One-hot activations pick single dequantised weights: catches any transposed or permuted
    operand / accumulator layout exactly (values are exactly representable in fp16).  K = 64 runs the
    generic kernel, the multiples of 256 the main one (several k-stages, ragged M and N tiles)."""
    rng = np.random.default_rng(0)
    nib = rng.integers(0, 16, (n, k // 32, 32))
    qs = (nib[..., :16] | (nib[..., 16:] << 4)).astype(np.uint8)
    d = np.full((n, k // 32, 1), 0.5, np.float16).view(np.uint8)
    wq = np.concatenate([d, qs], axis=-1).reshape(n, -1)
    x = np.zeros((m, k), np.float32)
    cols = rng.integers(0, k, m)
    x[np.arange(m), cols] = 2.0
    got = _gemm(dev, wq, x)
    w = npref.q4_0_dequant(wq)
    assert np.array_equal(got, 2.0 * w[:, cols].T)


@pytest.mark.parametrize("m,k,n", [(1, 32, 1), (2, 64, 3), (63, 96, 65), (64, 128, 64), (65, 256, 129),
                                   (128, 512, 128), (129, 4096, 257), (512, 1024, 384), (1, 256, 1), (300, 768, 177),
                                   (16, 2048, 176), (17, 11008, 100)])
def test_gemm_shapes_vs_oracle(dev, m, k, n):
    wq, x = _case(m * 7 + k + n, m, k, n)
    ref = oracle.mul_mat_q4_0_f32(wq, x)
    emax, el2 = npref.rel_err(_gemm(dev, wq, x), ref)
    assert emax < TOL and el2 < TOL, (m, k, n, emax, el2)


def test_gemm_prefill_config(dev):
    m, k, n = 512, 4096, 11008
    wq, x = _case(3, m, k, n)
    got = _gemm(dev, wq, x)
    # every one of the 512 x 11008 outputs against dequantize-then-GEMM in f64 (numpy's matmul on the independent
    # vectorised dequantizer of tests/npref.py) ...
    full = x.astype(np.float64) @ npref.q4_0_dequant(wq).astype(np.float64).T
    emax, el2 = npref.rel_err(got, full)
    worst_col = float(np.max(np.max(np.abs(got - full), axis=0)) / np.max(np.abs(full)))
    print("prefill, all outputs: max_rel=%.3g l2_rel=%.3g (worst column %.3g)" % (emax, el2, worst_col))
    assert emax < TOL and el2 < TOL
    # ... and the C oracle on a column sample, which ties the numpy reference to the oracle at this size
    cols = np.random.default_rng(4).choice(n, 512, replace=False)
    ref = oracle.mul_mat_q4_0_f32(wq[cols], x)
    emax, el2 = npref.rel_err(full[:, cols], ref)
    assert emax < 1e-6 and el2 < 1e-6
    emax, el2 = npref.rel_err(got[:, cols], ref)
    assert emax < TOL and el2 < TOL
    # size-independent property at the full size: linearity in X (exact except where halving
    # pushes an fp16 activation into the subnormal range)
    got2 = _gemm(dev, wq, (0.5 * x).astype(np.float32))
    emax, el2 = npref.rel_err(got2, 0.5 * got)
    assert emax < 1e-6 and el2 < 1e-6
    # GEMM rows agree with the decode GEMV on the same activations
    wbuf, xbuf, ybuf = dev.upload(wq), dev.upload(x[7]), dev.alloc(n * 4)
    dev.dequantize_mul_mat_vec_q4_0(wbuf, xbuf, ybuf, k, n)
    yv = dev.download(ybuf, np.float32, n)
    emax, el2 = npref.rel_err(got[7], yv)
    assert emax < TOL and el2 < TOL
    for b in (wbuf, xbuf, ybuf):
        dev.free(b)


@pytest.mark.parametrize("m,k,n", [(512, 4096, 4096), (512, 11008, 4096), (512, 4096, 4112), (256, 4096, 8192)])
def test_gemm_narrow_matrices_at_full_size(dev, m, k, n):
    """The other prefill products of a LLaMA-7B layer (N = 4096), which run the narrower column tile (48 columns per
    workgroup instead of 96, chosen by how many workgroups that gives the device), and two more sizes: a column
    sample against the oracle and linearity at the full size."""
    wq, x = _case(m + k + n, m, k, n)
    got = _gemm(dev, wq, x)
    cols = np.random.default_rng(5).choice(n, 192, replace=False)
    cols[:3] = (0, n - 1, n // 2)
    emax, el2 = npref.rel_err(got[:, cols], oracle.mul_mat_q4_0_f32(wq[cols], x))
    assert emax < TOL and el2 < TOL, (emax, el2)
    got2 = _gemm(dev, wq, (0.5 * x).astype(np.float32))
    emax, el2 = npref.rel_err(got2, 0.5 * got)
    assert emax < 1e-6 and el2 < 1e-6


def test_gemm_argument_errors(dev):
    from galois_amd import GaloisHipError
    buf = dev.alloc(4096)
    for args, code in (((buf, buf, buf, 48, 1, 1), -2), ((buf, buf, buf, 32, 0, 1), -2),
                       ((buf, buf, buf, 32, 1, 0), -2), ((buf, None, buf, 32, 1, 1), -1),
                       ((buf.view(1), buf, buf, 32, 1, 1), -3), ((buf, buf.view(4), buf, 32, 1, 1), -3)):
        with pytest.raises(GaloisHipError) as ei:
            dev.mul_mat_q4_0_f32(*args)
        assert ei.value.status == code
    dev.free(buf)
