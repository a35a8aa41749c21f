"""Causal attention of many query rows in one launch (galois_hip_attn_prefill_f32 / _f16kv) through the C ABI.

The checker is the op sequence it replaces, restated in f64 numpy on the same inputs: per head scores = K q * scale
over the keys 0 .. n_past + m of query m, soft_max, out = V^T p (for an f16 cache on the cache's own rounded values).
The kernel's products take fp16 operands (q * scale * log2 e, keys, values, probabilities) with f32 sums: the bar is
2e-3 of the largest output magnitude for unit-variance inputs (scores of a few units), the header's statement, and
5e-3 where the scores reach +-100: rounding q and k to fp16 moves a score by about 2^-11 of its terms' size, and the
exponential turns that absolute error into a relative one of the probabilities; the panel output is additionally the f32 output of the
same call rounded to fp16.  Rows are independent of how the launch is cut into workgroups: the two workgroup shapes
(64 or 128 queries) are compared with each other through a row count that selects the larger one, and the larger
one is also the shape of the case of 1024 rows behind 1024 cached positions.
"""
import numpy as np
import pytest

from tests import npref

pytestmark = pytest.mark.gpu
TOL = 2e-3
D = 128


def _reference(q, kc, vc, n_head, n_past, scale):
    n = q.shape[0]
    out = np.zeros((n, n_head * D))
    keys = np.arange(n_past + n)
    visible = keys[None, :] <= (n_past + np.arange(n))[:, None]
    for h in range(n_head):
        sl = slice(h * D, (h + 1) * D)
        s = (q[:, sl].astype(np.float64) @ kc[:n_past + n, sl].astype(np.float64).T) * scale
        s = np.where(visible, s, -np.inf)
        p = np.exp(s - s.max(axis=1, keepdims=True))
        p /= p.sum(axis=1, keepdims=True)
        out[:, sl] = p @ vc[:n_past + n, sl].astype(np.float64)
    return out


def _untile(raw, m, k):
    m_pad = (m + 15) // 16 * 16
    t = raw.view(np.float16).reshape(m_pad // 16, k // 32, 4, 16, 8)
    return t.transpose(0, 3, 1, 2, 4).reshape(m_pad, k)


def _inputs(seed, n_head, n, n_past, n_ctx, kv_f16, spread=1.0):
    rng = np.random.default_rng(seed)
    e = n_head * D
    q = (rng.standard_normal((n, e)) * spread).astype(np.float32)
    kc = rng.standard_normal((n_ctx, e)).astype(np.float32)
    vc = rng.standard_normal((n_ctx, e)).astype(np.float32)
    # rows the call must not look at hold NaN: a key past n_past + n that leaks into a sum shows
    kc[n_past + n:] = np.nan
    vc[n_past + n:] = np.nan
    if kv_f16:
        kc, vc = kc.astype(np.float16), vc.astype(np.float16)
    return q, kc, vc


@pytest.mark.parametrize("kv_f16", [False, True])
@pytest.mark.parametrize("n_head,n,n_past", [(2, 1, 0), (2, 20, 0), (3, 77, 19), (32, 512, 0), (4, 64, 1), (2, 65, 31),
                                             (1, 130, 700), (8, 300, 1000), (32, 1024, 1024)])
def test_attention_of_many_rows_against_the_op_sequence_in_f64(dev, n_head, n, n_past, kv_f16):
    e = n_head * D
    n_ctx = n_past + n + 5
    q, kc, vc = _inputs(n_head * 1000 + n + n_past, n_head, n, n_past, n_ctx, kv_f16)
    scale = float(np.float32(1.0) / np.sqrt(np.float32(D)))
    ref = _reference(q, kc, vc, n_head, n_past, scale)
    qb, kb, vb = dev.upload(q), dev.upload(kc), dev.upload(vc)
    ob = dev.upload(np.full((n, e), 3.25, np.float32))
    dev.attn_prefill(qb, kb, vb, ob, None, n_head, D, n, n_past, scale, kv_f16)
    got = dev.download(ob, np.float32, n * e).reshape(n, e)
    assert np.all(np.isfinite(got))
    emax, el2 = npref.rel_err(got, ref)
    assert emax < TOL and el2 < TOL, (emax, el2)
    nbytes = (n + 15) // 16 * 16 * e * 2      # the panel's tiles need only whole groups of 32 columns
    pb = dev.alloc(nbytes)
    dev.upload(np.full(nbytes // 4, 7.5, np.float32), pb)
    dev.attn_prefill(qb, kb, vb, None, pb, n_head, D, n, n_past, scale, kv_f16)
    panel = _untile(dev.download(pb, np.uint8, nbytes), n, e)
    assert np.array_equal(panel[:n].view(np.uint16), got.astype(np.float16).view(np.uint16)), "the panel is the f32 result rounded"
    assert np.all(panel[n:] == 0), "rows past n are zero in the panel"
    for b in (qb, kb, vb, ob, pb):
        dev.free(b)


def test_peaked_scores_and_the_first_row(dev):
    """Queries eight times larger (scores of +-100 and more, probabilities that are a few keys'): the running maximum
    and the rescaling carry the result, to the wider bar of such scores; and row 0 of an empty context is exactly V[0] rounded to fp16."""
    n_head, n, n_past = 2, 100, 0
    q, kc, vc = _inputs(77, n_head, n, n_past, n, False, spread=8.0)
    scale = float(np.float32(1.0) / np.sqrt(np.float32(D)))
    ref = _reference(q, kc, vc, n_head, n_past, scale)
    qb, kb, vb = dev.upload(q), dev.upload(kc), dev.upload(vc)
    ob = dev.alloc(n * n_head * D * 4)
    dev.attn_prefill(qb, kb, vb, ob, None, n_head, D, n, n_past, scale)
    got = dev.download(ob, np.float32, n * n_head * D).reshape(n, -1)
    emax, el2 = npref.rel_err(got, ref)
    assert emax < 5e-3 and el2 < TOL, (emax, el2)
    assert np.array_equal(got[0], vc[0].astype(np.float16).astype(np.float32))
    for b in (qb, kb, vb, ob):
        dev.free(b)


def test_rows_do_not_depend_on_the_workgroup_shape(dev):
    """8 heads x 8400 rows select 128 queries per workgroup, the first 4096 of them alone 64 (on 256 CUs): a row's
    result is the same in both launches bit for bit, since a row's walk over its keys is the same."""
    n_head, n = 8, 8400
    rng = np.random.default_rng(5)
    e = n_head * D
    q = rng.standard_normal((n, e)).astype(np.float32)
    kc = rng.standard_normal((n, e)).astype(np.float16)
    vc = rng.standard_normal((n, e)).astype(np.float16)
    scale = 0.088
    qb, kb, vb = dev.upload(q), dev.upload(kc), dev.upload(vc)
    ob, ob2 = dev.alloc(n * e * 4), dev.alloc(4096 * e * 4)
    dev.attn_prefill(qb, kb, vb, ob, None, n_head, D, n, 0, scale, True)
    dev.attn_prefill(qb, kb, vb, ob2, None, n_head, D, 4096, 0, scale, True)
    big = dev.download(ob, np.float32, n * e).reshape(n, e)
    small = dev.download(ob2, np.float32, 4096 * e).reshape(4096, e)
    assert np.array_equal(big[:4096], small)
    # the last rows against f64, without the full 8400 x 8400 reference
    for m in (8399, 4097):
        for h in range(n_head):
            sl = slice(h * D, (h + 1) * D)
            s = (kc[:m + 1, sl].astype(np.float64) @ q[m, sl].astype(np.float64)) * scale
            p = np.exp(s - s.max())
            p /= p.sum()
            o = p @ vc[:m + 1, sl].astype(np.float64)
            assert np.max(np.abs(big[m, sl] - o)) < TOL * max(np.max(np.abs(o)), 0.05)
    for b in (qb, kb, vb, ob, ob2):
        dev.free(b)


def test_refusals(dev):
    import galois_amd as ga
    b = dev.alloc(1 << 16)
    for out, panel in ((b, b), (None, None)):                     # both outputs, neither
        with pytest.raises(ga.GaloisHipError):
            dev.attn_prefill(b, b, b, out, panel, 2, D, 4, 0, 0.1)
    with pytest.raises(ga.GaloisHipError):
        dev.attn_prefill(b, b, b, b, None, 2, 64, 4, 0, 0.1)      # heads of 64
    with pytest.raises(ga.GaloisHipError):
        dev.attn_prefill(b, b, b, b, None, 2, D, 0, 0, 0.1)       # no rows
    with pytest.raises(ga.GaloisHipError):
        dev.attn_prefill(b, b, b, b, None, 2, D, 4, -1, 0.1)      # negative n_past
    with pytest.raises(ga.GaloisHipError):
        dev.attn_prefill(b.ptr + 4, b, b, b, None, 2, D, 4, 0, 0.1)   # unaligned q
    dev.free(b)
