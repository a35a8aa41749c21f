"""CPU test of the activation preparation used by the decode GEMV (gemv_xprep.h).

The header is plain C++; it is compiled here with g++ and checked against a direct
Python model of the arithmetic it claims: block-scaled fixed point in balanced base 16,
laid out so that dot8(weights ^ 0x88888888, plane_l) summed with weights 16^l equals the
exact integer dot product of (q - 8) with the fixed-point activations.
"""
import ctypes as C
import os
import subprocess

import numpy as np
import pytest

import oracle
from tests import npref

HERE = os.path.dirname(os.path.abspath(__file__))


@pytest.fixture(scope="module")
def shim(tmp_path_factory):
    so = str(tmp_path_factory.mktemp("xprep") / "xprep_shim.so")
    subprocess.check_call(["g++", "-O2", "-std=c++17", "-shared", "-fPIC", "-o", so,
                           os.path.join(HERE, "xprep_shim.cc")])
    return C.CDLL(so)


def _planes(shim, L, x64):
    x64 = np.ascontiguousarray(x64, np.float32)
    planes = np.zeros((L, 8), np.uint32)
    scales = np.zeros(2, np.float32)
    shim.xprep_slot_planes(L, x64.ctypes.data_as(C.c_void_p), planes.ctypes.data_as(C.c_void_p),
                           scales.ctypes.data_as(C.c_void_p))
    return planes, scales


def _sdigit(n):
    return n - 16 if n >= 8 else n


def test_transpose_is_a_nibble_transpose(shim):
    rng = np.random.default_rng(0)
    a = rng.integers(0, 2 ** 32, 8, dtype=np.uint64).astype(np.uint32)
    out = np.zeros(8, np.uint32)
    shim.xprep_transpose(a.ctypes.data_as(C.c_void_p), out.ctypes.data_as(C.c_void_p))
    for j in range(8):
        for l in range(8):
            assert (int(out[l]) >> (4 * j)) & 0xF == (int(a[j]) >> (4 * l)) & 0xF


def test_group_index_covers_each_activation_once(shim):
    seen = sorted(shim.xprep_group_x_index(g, j) for g in range(8) for j in range(8))
    assert seen == list(range(64))


@pytest.mark.parametrize("L", [4, 5, 6])
def test_planes_reconstruct_fixed_point_activations(shim, L):
    rng = np.random.default_rng(L)
    xbits = 4 * L - 2
    for scale in (1.0, 1e-3, 37.0, 1e-30, 1e30):
        x = (rng.standard_normal(64) * scale).astype(np.float32)
        planes, scales = _planes(shim, L, x)
        for blk in range(2):
            amax = float(np.max(np.abs(x[32 * blk:32 * blk + 32])))
            e = int(np.floor(np.log2(amax)))
            assert scales[blk] == np.float32(2.0 ** (e - xbits + 1))
        for g in range(8):
            for j in range(8):
                k = shim.xprep_group_x_index(g, j)
                X = sum(_sdigit((int(planes[l, g]) >> (4 * j)) & 0xF) * 16 ** l for l in range(L))
                s = float(scales[k // 32])
                # exact RNE of x / s on the integer grid
                assert X == int(np.rint(np.float64(x[k]) / s)), (g, j)
                assert abs(X * s - float(x[k])) <= 0.5 * s


def test_integer_dot_identity_and_accuracy(shim):
    """Emulates the kernel's arithmetic on the CPU for whole rows and compares with the oracle."""
    rng = np.random.default_rng(9)
    k, n, L = 256, 5, 6
    w = (rng.standard_normal((n, k)) * 0.02).astype(np.float32)
    x = rng.standard_normal(k).astype(np.float32)
    wq = oracle.quantize_q4_0(w)
    d, nib = npref.q4_0_unpack(wq)  # nib [n, nb, 32] in weight order
    y = np.zeros(n, np.float64)
    for s in range(k // 64):
        planes, scales = _planes(shim, L, x[64 * s:64 * s + 64])
        # fixed-point activations in weight order, rebuilt from the planes
        X = np.zeros(64, np.int64)
        for g in range(8):
            for j in range(8):
                X[shim.xprep_group_x_index(g, j)] = sum(
                    _sdigit((int(planes[l, g]) >> (4 * j)) & 0xF) * 16 ** l for l in range(L))
        for blk in range(2):
            t = (nib[:, 2 * s + blk, :] - 8).astype(np.int64) @ X[32 * blk:32 * blk + 32]
            assert np.all(np.abs(t) < 2 ** 31)
            y += d[:, 2 * s + blk].astype(np.float64) * float(scales[blk]) * t
    emax, el2 = npref.rel_err(y, oracle.mul_mat_q4_0_f32(wq, x))
    assert emax < 2e-6 and el2 < 2e-6


def test_special_blocks(shim):
    # all-zero block: scale 0, all planes 0; unit activation: exact power-of-two fixed point
    planes, scales = _planes(shim, 6, np.zeros(64, np.float32))
    assert np.all(planes == 0) and np.all(scales == 0)
    x = np.zeros(64, np.float32)
    x[5] = 1.0
    planes, scales = _planes(shim, 6, x)
    assert scales[0] == np.float32(2.0 ** -21) and scales[1] == 0
    # non-finite activation poisons its block's scale
    x[40] = np.inf
    planes, scales = _planes(shim, 6, x)
    assert np.isnan(scales[1]) and scales[0] == np.float32(2.0 ** -21)


# ---- corrections: what the fixed point rounds away comes back for blocks that a few activations dominate

def _digits_to_int(planes, L, g, j):
    return sum(_sdigit((int(planes[l, g]) >> (4 * j)) & 0xF) * 16 ** l for l in range(L))


def _emulate_gemv(shim, wq, x):
    """The kernel's arithmetic for whole rows on the CPU: exact integer dots of (q - 8) with the planes and with
    the correction planes, each times its power-of-two scale and the block's d (accumulated in f64 here)."""
    L, CL = 5, shim.xprep_corr_limbs()
    shim.xprep_slot_full.restype = None
    d, nib = npref.q4_0_unpack(wq)
    n, k = wq.shape[0], x.size
    y = np.zeros(n, np.float64)
    flagged = 0
    for s in range(k // 64):
        x64 = np.ascontiguousarray(x[64 * s:64 * s + 64], np.float32)
        planes, scales = np.zeros((L, 8), np.uint32), np.zeros(2, np.float32)
        planes2, scales2 = np.zeros((CL, 8), np.uint32), np.zeros(2, np.float32)
        shim.xprep_slot_full(x64.ctypes.data_as(C.c_void_p), planes.ctypes.data_as(C.c_void_p),
                             scales.ctypes.data_as(C.c_void_p), planes2.ctypes.data_as(C.c_void_p),
                             scales2.ctypes.data_as(C.c_void_p))
        X, X2 = np.zeros(64, np.int64), np.zeros(64, np.int64)
        for g in range(8):
            for j in range(8):
                X[shim.xprep_group_x_index(g, j)] = _digits_to_int(planes, L, g, j)
                X2[shim.xprep_group_x_index(g, j)] = _digits_to_int(planes2, CL, g, j)
        for blk in range(2):
            q = (nib[:, 2 * s + blk, :] - 8).astype(np.int64)
            t, t2 = q @ X[32 * blk:32 * blk + 32], q @ X2[32 * blk:32 * blk + 32]
            assert np.all(np.abs(t) < 2 ** 31) and np.all(np.abs(t2) < 2 ** 31)
            dd = d[:, 2 * s + blk].astype(np.float64)
            y += dd * float(scales[blk]) * t + dd * float(scales2[blk]) * t2
            flagged += scales2[blk] != 0
            # what the two fixed-point parts leave behind, against the documented bound
            xb = x64[32 * blk:32 * blk + 32].astype(np.float64)
            left = xb - X[32 * blk:32 * blk + 32] * float(scales[blk]) - X2[32 * blk:32 * blk + 32] * float(scales2[blk])
            top = 2.0 ** np.floor(np.log2(np.max(np.abs(xb)))) if np.any(xb) else 0.0
            low = np.abs(xb) < top
            if scales[blk] != 0:
                assert np.all(np.abs(left[~low]) <= 2.0 ** -18 * np.abs(xb[~low]))
            if scales2[blk] == 0:
                rest = np.arange(32) != int(np.argmax(np.abs(xb)))
                assert np.sum(np.abs(left[rest])) <= 2.0 ** -13 * np.sum(np.abs(xb[rest]))
            else:
                sel = low if scales[blk] != 0 else np.ones(32, bool)
                assert np.all(np.abs(left[sel]) <= 0.5 * float(scales2[blk]))
                assert float(scales2[blk]) <= 2.0 ** -12 * max(np.max(np.abs(xb[sel])), float(scales[blk]) / 2)
    return y, flagged


def test_residual_is_exact(shim):
    shim.xprep_residual.restype = C.c_float
    shim.xprep_residual.argtypes = [C.c_float, C.c_float, C.c_float]
    rng = np.random.default_rng(3)
    for e in (-20, 0, 17):
        scale = 2.0 ** (e - 18)
        for x in np.concatenate([rng.standard_normal(200) * 2.0 ** e, rng.standard_normal(200) * 2.0 ** (e - 25),
                                 [0.0, scale / 2, -scale / 2, 1.5 * scale, 2.0 ** e]]).astype(np.float32):
            X = float(np.rint(np.float64(x) / scale))  # ties to even, like the kernel's magic-number rounding
            assert shim.xprep_residual(float(x), 1.0 / scale, scale) == np.float32(np.float64(x) - X * scale)
    assert shim.xprep_residual(3.0e-39, 0.0, 0.0) == np.float32(3.0e-39)  # a block without a grid keeps all of x


def _set_nibble(wq, col, value):
    b, j = divmod(col, 32)
    byte = b * 18 + 2 + (j % 16)
    if j < 16:
        wq[:, byte] = (wq[:, byte] & 0xF0) | value
    else:
        wq[:, byte] = (wq[:, byte] & 0x0F) | (value << 4)


@pytest.mark.parametrize("log2mag", [0, 6, 12, 18, 24])
@pytest.mark.parametrize("zero_weight", [False, True])
def test_emulated_gemv_with_outlier_activations(shim, log2mag, zero_weight):
    """One activation per block 2^log2mag times the others; with zero_weight it meets weight 0 in every row, so the
    rows consist of the small activations alone.  1e-4 of sum |w||x| row by row, and of max |ref| overall."""
    rng = np.random.default_rng(40 + log2mag)
    k, n = 512, 24
    wq = oracle.quantize_q4_0((rng.standard_normal((n, k)) * 0.02).astype(np.float32)).copy()
    x = rng.standard_normal(k).astype(np.float32)
    for b in range(k // 32):
        col = b * 32 + (7 * b + 3) % 32
        x[col] = np.float32((1.0 if b % 2 else -1.0) * 2.0 ** log2mag * (1.0 + 0.37 * (b % 5)))
        if zero_weight:
            _set_nibble(wq, col, 8)
    y, flagged = _emulate_gemv(shim, wq, x)
    w = npref.q4_0_dequant(wq).astype(np.float64)
    ref = w @ x.astype(np.float64)
    assert flagged == (k // 32 if log2mag >= 6 else 0)
    assert np.max(np.abs(y - ref) / (np.abs(w) @ np.abs(x.astype(np.float64)))) < 1e-4
    assert np.max(np.abs(y - ref)) / np.max(np.abs(ref)) < 1e-4


def test_emulated_gemv_plain_vectors_need_no_correction(shim):
    rng = np.random.default_rng(50)
    k, n = 1024, 8
    wq = oracle.quantize_q4_0((rng.standard_normal((n, k)) * 0.02).astype(np.float32))
    for x in (rng.standard_normal(k), rng.uniform(-1, 1, k), np.eye(k)[5], np.zeros(k), np.ones(k) * 0.1):
        x = x.astype(np.float32)
        y, flagged = _emulate_gemv(shim, wq, x)
        assert flagged == 0
        ref = npref.q4_0_dequant(wq).astype(np.float64) @ x.astype(np.float64)
        assert np.max(np.abs(y - ref)) <= 1e-5 * max(np.max(np.abs(ref)), 1e-30)
