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
