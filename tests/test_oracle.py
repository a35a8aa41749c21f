"""Pins the CPU oracle (oracle/galois_oracle.c) WITHOUT the reference's help.

galois's own tests assert nothing for this path, so every function of the oracle is
pinned here by (a) the hand-derived vectors in tests/golden/kat.json, (b) an
independent vectorised numpy restatement (tests/npref.py) or a library routine
(numpy float16, numpy float64 matmul, scipy softmax), and (c) invariants chosen so
that a dropped term, wrong nibble order, wrong sign or transposed operand fails.
"""
import json
import os

import numpy as np
import pytest
import scipy.special

import oracle
from tests import npref

KAT = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "kat.json")))


def _arr(x):
    return np.array([float(v) for v in x], np.float32)


# ----------------------------------------------------------------------------- f16
def test_f16_to_f32_exhaustive():
    h = np.arange(65536, dtype=np.uint16)
    got = oracle.f16_to_f32(h)
    ref = h.view(np.float16).astype(np.float32)
    assert np.array_equal(got.view(np.uint32)[~np.isnan(ref)], ref.view(np.uint32)[~np.isnan(ref)])
    assert np.all(np.isnan(got[np.isnan(ref)]))


def test_f32_to_f16_rne_against_numpy():
    rng = np.random.default_rng(1)
    # every half value, the midpoints between neighbours, and one ulp(f32) either side
    h = np.arange(0x7C00, dtype=np.uint16)
    lo = h.view(np.float16).astype(np.float32)
    hi = (h + 1).astype(np.uint16).view(np.float16).astype(np.float32)
    mid = ((lo.astype(np.float64) + hi.astype(np.float64)) / 2).astype(np.float32)
    pts = np.concatenate([lo, mid, np.nextafter(mid, np.float32(0)), np.nextafter(mid, np.float32(np.inf)),
                          rng.standard_normal(200000).astype(np.float32) * np.float32(100),
                          rng.standard_normal(200000).astype(np.float32) * np.float32(1e-6),
                          np.array([65504, 65519.99, 65520, 1e9, 2.0 ** -25, 2.0 ** -24, 0.0], np.float32)])
    pts = np.concatenate([pts, -pts])
    with np.errstate(over="ignore"):
        ref = pts.astype(np.float16).view(np.uint16)
    assert np.array_equal(oracle.f32_to_f16(pts), ref)


# ----------------------------------------------------------------------------- Q4_0 layout / dequant
def test_block_sizes():
    assert oracle.lib().orc_sizeof_block_q4_0() == 18
    assert oracle.lib().orc_sizeof_block_q8_0() == 34


def test_dequant_kat_layout():
    c = KAT["layout_ramp"]
    got = oracle.dequantize_q4_0(np.array(c["block"], np.uint8))
    assert np.array_equal(got, _arr(c["values"]))


def test_dequant_bruteforce_nibbles_and_scales():
    # every nibble value in every position x a spread of f16 scales incl. negative, subnormal
    scales = np.array([0x3C00, 0xBC00, 0x0001, 0x8001, 0x03FF, 0x7BFF, 0xFBFF, 0x2E66, 0x0000, 0x1234],
                      np.uint16)
    for dbits in scales:
        d = np.array([dbits], np.uint16).view(np.float16).astype(np.float32)[0]
        for pos in range(32):
            for nib in range(16):
                qs = np.full(16, 0x88, np.uint8)
                j = pos % 16
                qs[j] = (qs[j] & 0xF0) | nib if pos < 16 else (qs[j] & 0x0F) | (nib << 4)
                blk = np.concatenate([np.array([dbits], np.uint16).view(np.uint8), qs])
                got = oracle.dequantize_q4_0(blk)
                exp = np.zeros(32, np.float32) * d
                exp[pos] = np.float32(nib - 8) * d
                assert np.array_equal(got, exp), (hex(dbits), pos, nib)


def test_dequant_matches_numpy():
    rng = np.random.default_rng(2)
    raw = rng.integers(0, 256, size=(7, 5 * 18), dtype=np.uint8)
    # keep the f16 scale finite
    raw.reshape(7, 5, 18)[..., 1] &= 0x7B
    assert np.array_equal(oracle.dequantize_q4_0(raw), npref.q4_0_dequant(raw))


# ----------------------------------------------------------------------------- Q4_0 quantizer
@pytest.mark.parametrize("name", sorted(KAT["quantize_q4_0"]))
def test_quantize_q4_0_kat(name):
    c = KAT["quantize_q4_0"][name]
    got = oracle.quantize_q4_0(_arr(c["x"]))
    assert got.tolist() == c["block"], c["why"]


def test_quantize_q4_0_matches_numpy_bytes():
    rng = np.random.default_rng(3)
    for scale in (0.02, 1.0, 1e-7, 3e4):
        x = (rng.standard_normal((64, 4096)) * scale).astype(np.float32)
        assert np.array_equal(oracle.quantize_q4_0(x), npref.q4_0_quantize(x)), scale
    # ties in |x|, exact .5 boundaries
    x = rng.integers(-8, 9, size=(512, 64)).astype(np.float32)
    assert np.array_equal(oracle.quantize_q4_0(x), npref.q4_0_quantize(x))


def test_quantize_q4_0_invariants():
    rng = np.random.default_rng(4)
    x = (rng.standard_normal((256, 32)) * 0.02).astype(np.float32)
    q = oracle.quantize_q4_0(x)
    d, nib = npref.q4_0_unpack(q)
    d = d[:, 0]
    nib = nib[:, 0, :]
    imax = np.argmax(np.abs(x), axis=1)
    r = np.arange(len(x))
    # the max-magnitude element always gets nibble 0 and dequantises to -8*d
    assert np.all(nib[r, imax] == 0)
    w = oracle.dequantize_q4_0(q)
    assert np.array_equal(w[r, imax], np.float32(-8) * d)
    # round trip error bound: half a step (+ f16 rounding of d) unless clamped to the top bin
    err = np.abs(w - x)
    step = np.abs(d)[:, None]
    clamped = nib == 15
    assert np.all(err[~clamped] <= (step * (0.5 + 2.0 ** -8) + 1e-12)[np.nonzero(~clamped)[0], 0])
    assert np.all(err[clamped] <= (step * (1.0 + 2.0 ** -8) + 1e-12)[np.nonzero(clamped)[0], 0])
    # determinism
    assert np.array_equal(q, oracle.quantize_q4_0(x.copy()))
    # sign flip of the whole block flips d and mirrors nothing else: values negate exactly
    # except where the +8.5 truncation is asymmetric; the dequantised max element still negates
    w2 = oracle.dequantize_q4_0(oracle.quantize_q4_0(-x))
    assert np.array_equal(w2[r, imax], -w[r, imax])


# ----------------------------------------------------------------------------- Q8_0 + CPU dot
@pytest.mark.parametrize("name", sorted(KAT["quantize_q8_0"]))
def test_quantize_q8_0_kat(name):
    c = KAT["quantize_q8_0"][name]
    got = oracle.quantize_q8_0(_arr(c["x"]))
    assert int(got[:2].view(np.uint16)[0]) == c["d_bits"]
    assert got[2:].view(np.int8).tolist() == c["q"]


def test_quantize_q8_0_matches_numpy():
    rng = np.random.default_rng(5)
    x = rng.standard_normal((33, 1024)).astype(np.float32)
    assert np.array_equal(oracle.quantize_q8_0(x), npref.q8_0_quantize(x))
    # the amax element maps to +-127
    d, q = npref.q8_0_unpack(oracle.quantize_q8_0(x))
    assert np.all(np.max(np.abs(q), axis=-1) == 127)


def test_vec_dot_integer_part_and_avx_equals_scalar():
    rng = np.random.default_rng(6)
    k = 4096
    w = (rng.standard_normal(k) * 0.02).astype(np.float32)
    x = rng.standard_normal(k).astype(np.float32)
    wq, xq = oracle.quantize_q4_0(w), oracle.quantize_q8_0(x)
    dw, nib = npref.q4_0_unpack(wq)
    dx, q8 = npref.q8_0_unpack(xq)
    sumi = np.sum((nib - 8) * q8, axis=-1)                      # exact integers
    ref = float(np.sum(sumi.astype(np.float64) * dw.astype(np.float64) * dx.astype(np.float64)))
    s = oracle.vec_dot_q4_0_q8_0(wq, xq, "scalar")
    a = oracle.vec_dot_q4_0_q8_0(wq, xq, "avx2")
    scale = float(np.sum(np.abs(sumi) * np.abs(dw) * np.abs(dx)))
    assert abs(s - ref) <= 1e-6 * scale
    assert abs(a - ref) <= 1e-6 * scale
    # KAT: ramp block (d=1) . all-ones Q8 block (d=1)  = sum of the ramp values = -16
    ramp = np.array(KAT["layout_ramp"]["block"], np.uint8)
    ones = np.concatenate([np.array([0x3C00], np.uint16).view(np.uint8), np.ones(32, np.uint8)])
    assert oracle.vec_dot_q4_0_q8_0(ramp, ones, "scalar") == -16.0
    assert oracle.vec_dot_q4_0_q8_0(ramp, ones, "avx2") == -16.0


def test_cpu_baseline_structure_and_distance_from_oracle():
    rng = np.random.default_rng(7)
    k, n, m = 256, 50, 3
    w = (rng.standard_normal((n, k)) * 0.02).astype(np.float32)
    x = rng.standard_normal((m, k)).astype(np.float32)
    wq = oracle.quantize_q4_0(w)
    xq = oracle.quantize_q8_0(x)
    for nth in (1, 4, 7):
        y = oracle.cpu_mul_mat_q4_0_f32(wq, x, nth)
        for mi in range(m):
            for ni in range(0, n, 7):
                assert y[mi, ni] == np.float32(oracle.vec_dot_q4_0_q8_0(wq[ni], xq[mi], "avx2"))
    # informational: the Q8_0 baseline differs from the dequant oracle by ~1e-2, not 1e-4
    ref = oracle.mul_mat_q4_0_f32(wq, x)
    _, l2 = npref.rel_err(y, ref)
    assert 1e-5 < l2 < 5e-2


# ----------------------------------------------------------------------------- matmul parity oracle
def test_gemv_kat():
    c = KAT["gemv"]
    wq = np.array(c["W"], np.uint8)
    for case in c["cases"]:
        assert oracle.mul_mat_q4_0_f32(wq, _arr(case["x"])).tolist() == case["y"]


def test_mul_mat_oracle_against_numpy_f64():
    rng = np.random.default_rng(8)
    k, n, m = 512, 37, 5
    wq = oracle.quantize_q4_0((rng.standard_normal((n, k)) * 0.02).astype(np.float32))
    x = rng.standard_normal((m, k)).astype(np.float32)
    w = npref.q4_0_dequant(wq).astype(np.float64)
    ref = x.astype(np.float64) @ w.T
    got = oracle.mul_mat_q4_0_f32(wq, x, nthreads=3)
    assert got.shape == (m, n)
    assert np.allclose(got, ref, rtol=0, atol=2e-7 * np.max(np.abs(ref)))
    # unit vectors return columns of the dequantised matrix exactly; all-0x88 weights give 0
    for kk in (0, 17, 511):
        e = np.zeros(k, np.float32)
        e[kk] = 1
        assert np.array_equal(oracle.mul_mat_q4_0_f32(wq, e), w[:, kk].astype(np.float32))
    z = np.tile(np.array([0x00, 0x3C] + [0x88] * 16, np.uint8), (4, k // 32))
    assert np.all(oracle.mul_mat_q4_0_f32(z, x) == 0)


def test_mul_mat_f32_against_numpy():
    rng = np.random.default_rng(9)
    a = rng.standard_normal((2, 7, 16)).astype(np.float32)
    b = rng.standard_normal((4, 3, 16)).astype(np.float32)
    got = oracle.mul_mat_f32(a, b)
    ref = np.einsum("hmk,hnk->hmn", b.astype(np.float64), np.repeat(a, 2, axis=0).astype(np.float64))
    assert np.allclose(got, ref, rtol=1e-6, atol=1e-6)
    # a strided (transposed) view of a: same numbers, different strides
    at = np.ascontiguousarray(a.transpose(0, 2, 1)).transpose(0, 2, 1)
    assert not at.flags.c_contiguous
    assert np.array_equal(oracle.mul_mat_f32(at, b), got)


# ----------------------------------------------------------------------------- row ops
def test_rms_norm():
    c = KAT["rms_norm"]
    got = oracle.rms_norm(np.array(c["x"], np.float32), c["eps"])
    assert np.allclose(got, np.array(c["y"]), rtol=1e-7, atol=0)
    rng = np.random.default_rng(10)
    x = rng.standard_normal((9, 4096)).astype(np.float32)
    assert np.allclose(oracle.rms_norm(x, 1e-6), npref.rms_norm(x, 1e-6), rtol=1e-7, atol=1e-9)
    wv = (1 + 0.1 * rng.standard_normal(4096)).astype(np.float32)
    got = oracle.mul(oracle.rms_norm(x, 1e-6), wv)
    assert np.allclose(got, npref.rms_norm(x, 1e-6, wv), rtol=3e-7, atol=1e-9)


def test_elementwise():
    rng = np.random.default_rng(11)
    x = rng.standard_normal((6, 64)).astype(np.float32)
    v = rng.standard_normal(64).astype(np.float32)
    assert np.array_equal(oracle.mul(x, v), x * v)
    assert np.array_equal(oracle.add(x, v), x + v)
    assert np.array_equal(oracle.scale(x, 0.25), x * np.float32(0.25))
    xd = x.astype(np.float64)
    assert np.allclose(oracle.silu(x), xd / (1 + np.exp(-xd)), rtol=1e-7, atol=1e-12)


def test_rope():
    c = KAT["rope"]
    x = np.array(c["x"], np.float32)
    got = oracle.rope(x, c["pos"], c["freq_scale"], c["p_delta_rows"], c["theta_scale"])
    assert np.allclose(got, np.array(c["y"]), rtol=1e-6, atol=1e-7)
    assert np.array_equal(got[0], x[0])  # pos 0 is the identity
    rng = np.random.default_rng(12)
    t, h, hd = 11, 4, 128
    x = rng.standard_normal((t, h, hd)).astype(np.float32)
    pos = np.arange(5, 5 + t, dtype=np.int32)
    ts = float(np.float32(10000.0) ** np.float32(-2.0 / hd))
    got = oracle.rope(x.reshape(t * h, hd), pos, 1.0, h, ts).reshape(t, h, hd)
    ref = npref.rope(x, pos, h)
    assert np.allclose(got, ref, rtol=0, atol=2e-6)
    # rotation preserves pair norms; rotating by a then b equals a+b (up to f32 storage rounding)
    n0 = x[..., 0::2] ** 2 + x[..., 1::2] ** 2
    n1 = got[..., 0::2].astype(np.float64) ** 2 + got[..., 1::2].astype(np.float64) ** 2
    assert np.allclose(n0, n1, rtol=1e-5, atol=1e-6)
    a = oracle.rope(x.reshape(t * h, hd), np.full(t, 3, np.int32), 1.0, h, ts)
    ab = oracle.rope(a, np.full(t, 4, np.int32), 1.0, h, ts)
    direct = oracle.rope(x.reshape(t * h, hd), np.full(t, 7, np.int32), 1.0, h, ts)
    assert np.allclose(ab, direct, rtol=0, atol=2e-6)


def test_soft_max():
    c = KAT["soft_max"]
    x = np.array([float(v) for v in c["x"]], np.float32)
    got = oracle.soft_max(x[None, :])[0]
    assert np.allclose(got, np.array(c["y"]), rtol=1e-6, atol=0)
    assert got[2] == 0.0
    rng = np.random.default_rng(13)
    x = (rng.standard_normal((17, 512)) * 3).astype(np.float32)
    ref = scipy.special.softmax(x.astype(np.float64), axis=-1)
    got = oracle.soft_max(x)
    assert np.allclose(got, ref, rtol=2e-7, atol=1e-12)
    assert np.allclose(got.sum(-1), 1, atol=1e-6)
    assert np.allclose(oracle.soft_max(x + np.float32(5)), got, rtol=1e-5, atol=1e-9)  # shift invariance
    # causal: row r of each head keeps columns <= n_past + r; row 0 with n_past 0 is one-hot
    xc = (rng.standard_normal((2 * 8, 8)) * 3).astype(np.float32)
    got = oracle.soft_max_causal(xc, 8, 0)
    for r in range(16):
        last = r % 8
        assert np.all(got[r, last + 1:] == 0)
        assert np.allclose(got[r, :last + 1], scipy.special.softmax(xc[r, :last + 1].astype(np.float64)),
                           rtol=1e-6)
    assert got[0, 0] == 1.0 and got[8, 0] == 1.0


def test_cpy_and_get_rows():
    rng = np.random.default_rng(14)
    # permute [ne0=6, ne1=4, ne2=3] -> contiguous copy of the (ne1 <-> ne2)-swapped view, like galois_cont
    x = rng.standard_normal((3, 4, 6)).astype(np.float32)          # numpy [ne2, ne1, ne0]
    dst = np.zeros((4, 3, 6), np.float32)                           # want dst[i1, i2, i0] = x[i2, i1, i0]
    # source viewed as [ne00=6, ne01=3, ne02=4] with strides of the swapped view
    oracle.cpy_f32(x, dst, x.size, 6, 3, (4, 6 * 4 * 4, 6 * 4), 6, 3, (4, 6 * 4, 6 * 3 * 4))
    assert np.array_equal(dst, x.transpose(1, 0, 2))
    h = np.zeros((3, 4, 6), np.float16)
    oracle.cpy_f32(x, h, x.size, 6, 4, (4, 24, 96), 6, 4, (2, 12, 48))
    assert np.array_equal(h, x.astype(np.float16))
    w = oracle.quantize_q4_0((rng.standard_normal((10, 64)) * 0.02).astype(np.float32))
    ids = np.array([7, 0, 7, 9], np.int32)
    assert np.array_equal(oracle.get_rows_q4_0(w, ids), npref.q4_0_dequant(w)[ids])


def test_rope_f32_angle_restatement_agrees_with_the_oracle():
    """npref.rope_f32_angles (the reference kernel's f32 angle) against the oracle's f64 angle: identical where the
    angle is exact in f32 (position 0, pair 0), and apart only by the rounding of the angle elsewhere."""
    rng = np.random.default_rng(12)
    h, hd = 4, 128
    ts = float(np.float32(10000.0) ** np.float32(-2.0 / hd))
    for p0, tol in ((0, 2e-6), (100, 3e-5), (2040, 6e-4)):
        pos = np.arange(p0, p0 + 5, dtype=np.int32)
        x = rng.standard_normal((5 * h, hd)).astype(np.float32)
        a, b = npref.rope_f32_angles(x, pos, 1.0, h, ts), oracle.rope(x, pos, 1.0, h, ts)
        assert np.max(np.abs(a - b)) < tol, (p0, np.max(np.abs(a - b)))
        assert np.max(np.abs(a[:, :2] - b[:, :2])) < 2e-6      # pair 0: theta = pos exactly
