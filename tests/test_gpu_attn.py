"""GPU parity of the fused decode-step attention (through the C ABI) against the CPU oracle's op sequence:
rope(q), rope(k), append k and v to the caches, scores = K^T q, scale, soft_max, out = V p.

Tolerances.  The rotation angles are f32 on the GPU (the reference's formula) and f64 in the oracle, which at
positions near 2000 moves q and k by up to ~1e-4 (the tolerance of the rope_f32 parity test); against the
all-oracle sequence the outputs therefore agree to 2e-4.  With the rotated q and k taken from the GPU's own
rope_f32, what is left is the order of the f32 sums (per 128-key split, then across splits, exp relative to
split maxima first): 1e-5 relative to the largest output.  The appended cache rows equal rope_f32's output
and v bit for bit.
"""
import numpy as np
import pytest

import oracle
from galois_amd import GaloisHipError
from tests import npref

pytestmark = pytest.mark.gpu
TOL = 1e-5
TOL_ROPE = 2e-4


def _gpu_rope(dev, x, H, D, n_past, fs, ts):
    xb, yb, pb = dev.upload(x), dev.alloc(x.nbytes), dev.upload(np.array([n_past], np.int32))
    dev.rope_f32(xb, yb, D, H, pb, fs, H, ts)
    y = dev.download(yb, np.float32, x.size)
    for b in (xb, yb, pb):
        dev.free(b)
    return y


def _ref(q, k, v, kc, vc, H, D, n_past, fs, ts, scale, rotated=None):
    """The op sequence on the oracle; updates kc / vc (arrays [n_ctx, H*D]) in place; returns out [H*D].
    rotated = (rope(q), rope(k)) replaces the oracle's own rotation."""
    pos = np.array([n_past], np.int32)
    qr = oracle.rope(q.reshape(H, D), pos, fs, H, ts) if rotated is None else rotated[0].reshape(H, D)
    kr = oracle.rope(k.reshape(H, D), pos, fs, H, ts) if rotated is None else rotated[1].reshape(H, D)
    kc[n_past] = kr.reshape(-1)
    vc[n_past] = v
    L = n_past + 1
    kview = kc[:L].reshape(L, H, D).transpose(1, 0, 2)               # [H, L, D]: a strided view of the cache
    s = oracle.mul_mat_f32(kview, qr.reshape(H, 1, D))                # [H, 1, L]
    p = oracle.soft_max(oracle.scale(s, scale).reshape(H, L))
    vview = vc[:L].reshape(L, H, D).transpose(1, 2, 0)               # [H, D, L]
    return oracle.mul_mat_f32(vview, p.reshape(H, 1, L)).reshape(-1)


def _run(dev, q, k, v, kc, vc, H, D, n_past, fs, ts, scale):
    bufs = [dev.upload(a) for a in (q, k, v, kc, vc)]
    out = dev.alloc(H * D * 4 + 64)
    dev.upload(np.full(H * D + 16, 7.5, np.float32), out)
    pos = dev.upload(np.array([n_past], np.int32))
    dev.attn_decode_f32(bufs[0], bufs[1], bufs[2], bufs[3], bufs[4], out, H, D, n_past, pos, fs, ts, scale)
    o = dev.download(out, np.float32, H * D + 16)
    assert np.all(o[H * D:] == 7.5), "wrote past the end of out"
    kc_g = dev.download(bufs[3], np.float32, kc.shape)
    vc_g = dev.download(bufs[4], np.float32, vc.shape)
    for b in bufs + [out, pos]:
        dev.free(b)
    return o[:H * D], kc_g, vc_g


@pytest.mark.parametrize("H,D,n_ctx,n_past", [(32, 128, 2048, 2047), (32, 128, 2048, 0), (32, 128, 300, 127),
                                              (32, 128, 300, 128), (32, 128, 300, 129), (3, 128, 700, 511),
                                              (2, 64, 64, 37), (5, 64, 1000, 999), (1, 64, 130, 1),
                                              # more than 16 splits: the merge that keeps its weights in LDS
                                              # (17, 40 and 313 splits; past 256 its loops go round twice)
                                              (32, 128, 2049, 2048), (8, 128, 5001, 5000), (2, 64, 40001, 40000)])
def test_attn_decode_matches_the_op_sequence(dev, H, D, n_ctx, n_past):
    rng = np.random.default_rng(H * 1000 + D + n_past)
    E = H * D
    q, k, v = (rng.standard_normal(E).astype(np.float32) for _ in range(3))
    kc = rng.standard_normal((n_ctx, E)).astype(np.float32)
    vc = rng.standard_normal((n_ctx, E)).astype(np.float32)
    fs, ts, scale = 1.0, float(np.float32(10000.0) ** np.float32(-2.0 / D)), 1.0 / np.sqrt(D)
    got, kc_g, vc_g = _run(dev, q, k, v, kc, vc, H, D, n_past, fs, ts, scale)
    kc_ref, vc_ref = kc.copy(), vc.copy()
    ref = _ref(q, k, v, kc_ref, vc_ref, H, D, n_past, fs, ts, scale)
    emax, el2 = npref.rel_err(got, ref)
    assert emax < TOL_ROPE and el2 < TOL_ROPE, (emax, el2)
    qr, kr = _gpu_rope(dev, q, H, D, n_past, fs, ts), _gpu_rope(dev, k, H, D, n_past, fs, ts)
    ref = _ref(q, k, v, kc.copy(), vc.copy(), H, D, n_past, fs, ts, scale, rotated=(qr, kr))
    emax, el2 = npref.rel_err(got, ref)
    assert emax < TOL and el2 < TOL, (emax, el2)
    # exactly one cache row changed: row n_past = rope(k) as rope_f32 computes it, and v
    rows = np.arange(n_ctx) != n_past
    assert np.array_equal(kc_g[rows], kc[rows]) and np.array_equal(vc_g[rows], vc[rows])
    assert np.array_equal(vc_g[n_past], v)
    assert np.array_equal(kc_g[n_past], kr)
    emax, _ = npref.rel_err(kc_g[n_past], kc_ref[n_past])
    assert emax < TOL_ROPE * max(1.0, n_past / 2048.0)   # the f32 angle's rounding grows with the position


@pytest.mark.parametrize("H,D,n_ctx,n_past", [(32, 128, 2048, 2047), (32, 128, 300, 128), (2, 64, 64, 37), (5, 64, 1000, 0),
                                              (4, 128, 2200, 2100), (2, 64, 34000, 33500)])
def test_attn_decode_with_f16_caches(dev, H, D, n_ctx, n_past):
    """f16 caches: the appended rows are rope(k) and v rounded to nearest even, and the step computes with the
    rounded rows, like cpy_f32_f16 into the cache followed by the matmuls on its f16 contents."""
    rng = np.random.default_rng(H * 77 + D + n_past)
    E = H * D
    q, k, v = (rng.standard_normal(E).astype(np.float32) for _ in range(3))
    kc16 = rng.standard_normal((n_ctx, E)).astype(np.float16)
    vc16 = rng.standard_normal((n_ctx, E)).astype(np.float16)
    fs, ts, scale = 1.0, float(np.float32(10000.0) ** np.float32(-2.0 / D)), 1.0 / np.sqrt(D)
    bufs = [dev.upload(a) for a in (q, k, v, kc16, vc16)]
    out, pos = dev.alloc(E * 4), dev.upload(np.array([n_past], np.int32))
    dev.attn_decode_f16kv(bufs[0], bufs[1], bufs[2], bufs[3], bufs[4], out, H, D, n_past, pos, fs, ts, scale)
    got = dev.download(out, np.float32, E)
    kc_g, vc_g = dev.download(bufs[3], np.float16, kc16.shape), dev.download(bufs[4], np.float16, vc16.shape)
    qr, kr = _gpu_rope(dev, q, H, D, n_past, fs, ts), _gpu_rope(dev, k, H, D, n_past, fs, ts)
    rows = np.arange(n_ctx) != n_past
    assert np.array_equal(kc_g[rows], kc16[rows]) and np.array_equal(vc_g[rows], vc16[rows])
    assert np.array_equal(kc_g[n_past], kr.astype(np.float16)) and np.array_equal(vc_g[n_past], v.astype(np.float16))
    # the op sequence on the oracle over the f16 contents: rotated k and v already rounded as the cache holds them
    kc32, vc32 = kc16.astype(np.float32), vc16.astype(np.float32)
    ref = _ref(q, kr.astype(np.float16).astype(np.float32), v.astype(np.float16).astype(np.float32), kc32, vc32, H, D, n_past,
               fs, ts, scale, rotated=(qr, kr.astype(np.float16).astype(np.float32)))
    emax, el2 = npref.rel_err(got, ref)
    assert emax < TOL and el2 < TOL, (emax, el2)
    for b in bufs + [out, pos]:
        dev.free(b)


@pytest.mark.parametrize("H,D,n_ctx,n_past,f16", [(32, 128, 2048, 2047, False), (32, 128, 2100, 130, False),
                                                  (3, 64, 300, 299, False), (2, 128, 64, 0, False),
                                                  (32, 128, 2048, 2047, True), (5, 64, 700, 640, True)])
def test_head_major_caches_give_the_same_bits(dev, H, D, n_ctx, n_past, f16):
    """Caches kept [n_head][n_ctx][head_dim] hold the same elements at other addresses: the output and the cache
    contents equal those of the [n_ctx][n_head * head_dim] call bit for bit, for all three entry points."""
    rng = np.random.default_rng(H + D + n_past)
    E = H * D
    ct = np.float16 if f16 else np.float32
    q, k, v = (rng.standard_normal(E).astype(np.float32) for _ in range(3))
    kc = rng.standard_normal((n_ctx, E)).astype(ct)
    vc = rng.standard_normal((n_ctx, E)).astype(ct)
    hm = lambda c: np.ascontiguousarray(c.reshape(n_ctx, H, D).transpose(1, 0, 2))       # [H][n_ctx][D]
    fs, ts, scale = 1.0, float(np.float32(10000.0) ** np.float32(-2.0 / D)), 1.0 / np.sqrt(D)
    qb, kb, vb, pos = dev.upload(q), dev.upload(k), dev.upload(v), dev.upload(np.array([n_past], np.int32))
    calls = [dev.attn_decode_f16kv] if f16 else [dev.attn_decode_f32, dev.attn_decode_f32_static]
    for call in calls:
        res = []
        for layout in (0, n_ctx):
            kcb, vcb = dev.upload(hm(kc) if layout else kc), dev.upload(hm(vc) if layout else vc)
            out = dev.upload(np.full(E + 16, 7.5, np.float32))
            call(qb, kb, vb, kcb, vcb, out, H, D, n_past, pos, fs, ts, scale, layout)
            o = dev.download(out, np.float32, E + 16)
            kg, vg = dev.download(kcb, ct, (H, n_ctx, D) if layout else (n_ctx, E)), dev.download(vcb, ct, (H, n_ctx, D) if layout else (n_ctx, E))
            if layout:
                kg, vg = kg.transpose(1, 0, 2).reshape(n_ctx, E), vg.transpose(1, 0, 2).reshape(n_ctx, E)
            res.append((o, kg, vg))
            for b in (kcb, vcb, out):
                dev.free(b)
        for a, b in zip(*res):
            assert np.array_equal(a.view(np.uint8), b.view(np.uint8))
        assert np.all(res[1][0][E:] == 7.5) and np.all(np.isfinite(res[1][0][:E]))
    if n_past > 0:
        with pytest.raises(GaloisHipError) as ei:   # the capacity must exceed n_past
            calls[0](qb, kb, vb, qb, qb, qb, H, D, n_past, pos, fs, ts, scale, n_past)
        assert ei.value.status == -2
    for b in (qb, kb, vb, pos):
        dev.free(b)


def test_attn_decode_invariants(dev):
    """One key: the output is that key's value row whatever q is.  Equal keys: the mean of the values."""
    H, D, n_ctx = 4, 128, 512
    E = H * D
    rng = np.random.default_rng(3)
    q, k, v = (rng.standard_normal(E).astype(np.float32) for _ in range(3))
    ts = float(np.float32(10000.0) ** np.float32(-2.0 / D))
    got, _, _ = _run(dev, q, k, v, np.zeros((n_ctx, E), np.float32), np.zeros((n_ctx, E), np.float32), H, D, 0, 1.0, ts, 0.1)
    assert np.array_equal(got, v)
    # q = 0: every score is 0, softmax is uniform, out = mean of the value rows (300 keys: three splits)
    vc = rng.standard_normal((n_ctx, E)).astype(np.float32)
    got, _, vc_g = _run(dev, np.zeros(E, np.float32), k, v, rng.standard_normal((n_ctx, E)).astype(np.float32), vc, H, D,
                        299, 1.0, ts, 0.1)
    emax, el2 = npref.rel_err(got, vc_g[:300].astype(np.float64).mean(axis=0))
    assert emax < TOL and el2 < TOL


@pytest.mark.parametrize("L", [1500, 2700])   # 12 splits per head (merge in registers) and 22 (weights in LDS)
def test_attn_decode_repeated_calls_merge_fresh_partials(dev, L):
    """The splits of a head are merged by whichever workgroup finishes last, reading the other workgroups' records
    from a block that every call reuses: back-to-back calls with different values must each merge their own."""
    H, D = 32, 128
    rng = np.random.default_rng(21)
    fs, ts, scale = 1.0, float(np.float32(10000.0) ** np.float32(-2.0 / D)), float(1.0 / np.sqrt(D))
    kc = rng.standard_normal((L, H * D)).astype(np.float32)
    vc0 = rng.standard_normal((L, H * D)).astype(np.float32)
    q, k = (rng.standard_normal(H * D).astype(np.float32) for _ in range(2))
    pos = dev.upload(np.array([L - 1], np.int32))
    qb, kb, kcb = dev.upload(q), dev.upload(k), dev.upload(kc)
    outs, vbufs, vhost = [], [], []
    for i in range(12):            # values scaled differently per call, no synchronisation in between
        vc = (vc0 * np.float32(1.0 + i)).astype(np.float32)
        vhost.append(vc)
        vbufs.append((dev.upload(vc[L - 1].copy()), dev.upload(vc)))
        outs.append(dev.alloc(H * D * 4))
    for i in range(12):
        dev.attn_decode_f32(qb, kb, vbufs[i][0], kcb, vbufs[i][1], outs[i], H, D, L - 1, pos, fs, ts, scale)
    res = [dev.download(o, np.float32, H * D) for o in outs]
    for i in range(1, 12):         # the output is linear in the values
        err = np.max(np.abs(res[i] - res[0] * np.float32(1.0 + i))) / np.max(np.abs(res[i]))
        assert err <= 1e-6, (i, err)
    rot = (_gpu_rope(dev, q, H, D, L - 1, fs, ts), _gpu_rope(dev, k, H, D, L - 1, fs, ts))
    ref = _ref(q, k, vhost[0][L - 1].copy(), kc.copy(), vhost[0].copy(), H, D, L - 1, fs, ts, scale, rotated=rot)
    assert np.max(np.abs(res[0] - ref)) / np.max(np.abs(ref)) <= TOL


def test_attn_decode_argument_errors(dev):
    buf = dev.alloc(1 << 16)
    ok = [buf, buf, buf, buf, buf, buf, 2, 64, 0, buf, 1.0, 0.9, 0.1]
    for idx, val, code in ((7, 96, -5), (6, 0, -2), (8, -1, -2), (0, None, -1), (9, None, -1), (3, buf.view(4), -3),
                           (8, 40000000, -5)):
        args = list(ok)
        args[idx] = val
        if idx == 8 and val > 0:
            args[6] = 32
        with pytest.raises(GaloisHipError) as ei:
            dev.attn_decode_f32(*args)
        assert ei.value.status == code, (idx, val, ei.value.status)
    dev.free(buf)
