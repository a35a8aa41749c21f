"""GPU parity of the ops around the hot path (add / mul / scale / silu / cpy / get_rows / f32 matmul)."""
import numpy as np
import pytest

import oracle
from tests import npref

pytestmark = pytest.mark.gpu


def _out(dev, n, dtype=np.float32):
    b = dev.alloc(n * np.dtype(dtype).itemsize + 64)
    return b


@pytest.mark.parametrize("kx,ky", [(1, 1), (7, 7), (4096 * 5, 4096), (1000, 10), (33, 3), (11008, 11008)])
def test_add_mul_broadcast(dev, kx, ky):
    rng = np.random.default_rng(kx + ky)
    x, y = rng.standard_normal(kx).astype(np.float32), rng.standard_normal(ky).astype(np.float32)
    xb, yb, ob = dev.upload(x), dev.upload(y), _out(dev, kx)
    dev.add_f32(xb, yb, ob, kx, ky)
    assert np.array_equal(dev.download(ob, np.float32, kx), oracle.add(x, y))
    dev.mul_f32(xb, yb, ob, kx, ky)
    assert np.array_equal(dev.download(ob, np.float32, kx), oracle.mul(x, y))
    for b in (xb, yb, ob):
        dev.free(b)


@pytest.mark.parametrize("k", [11008, 11007, 3, 4, 1 << 20])   # multiples of 4 take the four-per-thread kernels
def test_scale_silu(dev, k):
    rng = np.random.default_rng(5)
    x, u = (rng.standard_normal(k) * 3).astype(np.float32), rng.standard_normal(k).astype(np.float32)
    xb, ub, ob = dev.upload(x), dev.upload(u), _out(dev, k)
    dev.scale_f32(xb, ob, 0.08838834764831845, k)
    assert np.array_equal(dev.download(ob, np.float32, k), oracle.scale(x, 0.08838834764831845))
    dev.silu_f32(xb, ob, k)
    emax, _ = npref.rel_err(dev.download(ob, np.float32, k), oracle.silu(x))
    assert emax < 1e-6
    dev.silu_mul_f32(xb, ub, ob, k)
    emax, _ = npref.rel_err(dev.download(ob, np.float32, k), oracle.silu(x).astype(np.float64) * u)
    assert emax < 1e-6
    for b in (xb, ub, ob):
        dev.free(b)


def test_cpy_strided_and_f16(dev):
    rng = np.random.default_rng(6)
    x = rng.standard_normal((3, 4, 6)).astype(np.float32)
    xb = dev.upload(x)
    # permuted view -> contiguous (galois_cont): dst[i1, i2, i0] = x[i2, i1, i0]
    ob = _out(dev, x.size)
    dev.cpy_f32(xb, ob, False, x.size, 6, 3, 4, 6 * 4 * 4, 6 * 4, 6, 3, 4, 6 * 4, 6 * 3 * 4)
    assert np.array_equal(dev.download(ob, np.float32, (4, 3, 6)), x.transpose(1, 0, 2))
    # f32 -> f16 contiguous (KV-cache write in an f16 cache)
    hb = _out(dev, x.size, np.float16)
    dev.cpy_f32(xb, hb, True, x.size, 6, 4, 4, 24, 96, 6, 4, 2, 12, 48)
    assert np.array_equal(dev.download(hb, np.float16, x.shape), x.astype(np.float16))
    # append one token's K vector at position p of a [L][4096] cache
    cache = np.zeros((8, 4096), np.float32)
    cb = dev.upload(cache)
    kvec = rng.standard_normal(4096).astype(np.float32)
    kb = dev.upload(kvec)
    dev.cpy_f32(kb, cb.view(5 * 4096 * 4), False, 4096, 4096, 1, 4, 4096 * 4, 4096 * 4, 4096, 1, 4, 4096 * 4, 4096 * 4)
    cache[5] = kvec
    assert np.array_equal(dev.download(cb, np.float32, cache.shape), cache)


def test_get_rows_q4_0(dev):
    rng = np.random.default_rng(7)
    w = oracle.quantize_q4_0((rng.standard_normal((100, 4096)) * 0.02).astype(np.float32))
    ids = np.array([99, 0, 5, 5, 42], np.int32)
    wb, ib, ob = dev.upload(w), dev.upload(ids), _out(dev, 5 * 4096)
    dev.get_rows_q4_0(wb, ib, ob, 4096, 5, 100)
    assert np.array_equal(dev.download(ob, np.float32, (5, 4096)), oracle.get_rows_q4_0(w, ids))
    # ids outside the table: nothing is read for them, their rows come back as NaN, the others as before
    bad = np.array([3, 100, -1, 2 ** 31 - 1, 7], np.int32)
    dev.upload(bad, ib)
    dev.get_rows_q4_0(wb, ib, ob, 4096, 5, 100)
    got = dev.download(ob, np.float32, (5, 4096))
    assert np.array_equal(got[[0, 4]], oracle.get_rows_q4_0(w, bad[[0, 4]])) and np.all(np.isnan(got[1:4]))


def test_attention_matmuls_over_a_kv_cache(dev):
    """QK^T and P.V of one decode step written with galois shapes: cache [L][n_head*head_dim] f32."""
    rng = np.random.default_rng(8)
    L, H, D = 300, 4, 128
    kc = rng.standard_normal((L, H * D)).astype(np.float32)
    vc = rng.standard_normal((L, H * D)).astype(np.float32)
    q = rng.standard_normal((H, 1, D)).astype(np.float32)
    kb, vb, qb = dev.upload(kc), dev.upload(vc), dev.upload(q)
    # scores[h][l] = sum_d K[l][h*D+d] * q[h][d]: a = view [ne0=D, ne1=L, ne2=H], strides (1, H*D, D)
    sb = _out(dev, H * L)
    dev.mul_mat_f32(kb, qb, sb, D, L, 1, H, H, 1, H * D, D)
    a_view = np.lib.stride_tricks.as_strided(kc, (H, L, D), (D * 4, H * D * 4, 4))
    ref = oracle.mul_mat_f32(a_view, q)
    got = dev.download(sb, np.float32, (H, 1, L))
    emax, _ = npref.rel_err(got, ref)
    assert emax < 1e-5
    # out[h][d] = sum_l V[l][h*D+d] * p[h][l]: a = view [ne0=L, ne1=D, ne2=H], strides (H*D, 1, D)
    p = oracle.soft_max((ref.reshape(H, L) / np.sqrt(D)).astype(np.float32)).reshape(H, 1, L)
    pb, ob = dev.upload(p), _out(dev, H * D)
    dev.mul_mat_f32(vb, pb, ob, L, D, 1, H, H, H * D, 1, D)
    v_view = np.lib.stride_tricks.as_strided(vc, (H, D, L), (D * 4, 4, H * D * 4))
    ref2 = oracle.mul_mat_f32(v_view, p)
    emax, _ = npref.rel_err(dev.download(ob, np.float32, (H, 1, D)), ref2)
    assert emax < 1e-5
    # broadcast of a over the batch (ne02 = 1, ne12 = 3) and M > 1
    a = rng.standard_normal((1, 9, 64)).astype(np.float32)
    b = rng.standard_normal((3, 2, 64)).astype(np.float32)
    ab, bb, ob2 = dev.upload(a), dev.upload(b), _out(dev, 3 * 2 * 9)
    dev.mul_mat_f32(ab, bb, ob2, 64, 9, 2, 1, 3, 1, 64, 9 * 64)
    emax, _ = npref.rel_err(dev.download(ob2, np.float32, (3, 2, 9)), oracle.mul_mat_f32(a, b))
    assert emax < 1e-5


def test_elementwise_argument_errors(dev):
    from galois_amd import GaloisHipError
    buf = dev.alloc(4096)
    for call, code in ((lambda: dev.add_f32(buf, buf, buf, 0, 1), -2), (lambda: dev.mul_f32(buf, None, buf, 4, 4), -1),
                       (lambda: dev.get_rows_q4_0(buf, buf, buf, 48, 1, 10), -2),
                       (lambda: dev.get_rows_q4_0(buf, buf, buf, 32, 1, 0), -2),
                       (lambda: dev.mul_mat_f32(buf, buf, buf, 4, 4, 1, 1, 1, 2, 2, 16), -5),
                       (lambda: dev.cpy_f32(buf, buf, False, 4, 2, 2, 3, 8, 16, 2, 2, 4, 8, 16), -3)):
        with pytest.raises(GaloisHipError) as ei:
            call()
        assert ei.value.status == code


@pytest.mark.parametrize("K,N,ne02,ne12,batch_fastest", [(128, 2048, 32, 32, True), (128, 37, 4, 4, True),
                                                         (64, 50, 1, 3, False), (32, 7, 2, 2, False),
                                                         (256, 19, 1, 1, False), (128, 21, 2, 6, True)])
def test_decode_scores_kernel_shapes(dev, K, N, ne02, ne12, batch_fastest):
    """M == 1 with rows contiguous along K: ragged row counts, both row orders, broadcast of a over the batch."""
    rng = np.random.default_rng(K + N)
    if batch_fastest:      # cache layout [N][ne02 * K]: batch stride K, row stride ne02 * K
        store = rng.standard_normal((N, ne02 * K)).astype(np.float32)
        a_view = np.lib.stride_tricks.as_strided(store, (ne02, N, K), (K * 4, ne02 * K * 4, 4))
        s1, s2 = ne02 * K, K
    else:
        store = rng.standard_normal((ne02, N, K)).astype(np.float32)
        a_view, s1, s2 = store, K, N * K
    b = rng.standard_normal((ne12, 1, K)).astype(np.float32)
    ab, bb, ob = dev.upload(store), dev.upload(b), _out(dev, ne12 * N)
    dev.mul_mat_f32(ab, bb, ob, K, N, 1, ne02, ne12, 1, s1, s2)
    emax, _ = npref.rel_err(dev.download(ob, np.float32, (ne12, 1, N)), oracle.mul_mat_f32(a_view, b))
    assert emax < 1e-5


@pytest.mark.parametrize("K,N,ne02,ne12", [(2048, 128, 32, 32), (1, 128, 2, 2), (15, 128, 2, 2), (17, 64, 1, 3),
                                           (63, 100, 3, 3), (64, 100, 3, 3), (65, 100, 3, 3), (5000, 36, 2, 4),
                                           (300, 4, 1, 1)])
def test_decode_values_kernel_shapes(dev, K, N, ne02, ne12):
    """M == 1 with a contiguous along N: one slab and many, ragged K, column tiles that end inside a wave,
    broadcast of a over the batch; launched twice so the second run meets the tickets the first one left."""
    rng = np.random.default_rng(K * 7 + N)
    store = rng.standard_normal((K, ne02 * N)).astype(np.float32)           # cache layout [K][ne02 * N]
    a_view = np.lib.stride_tricks.as_strided(store, (ne02, N, K), (N * 4, 4, ne02 * N * 4))
    ab, ob = dev.upload(store), _out(dev, ne12 * N)
    for rep in range(2):
        b = rng.standard_normal((ne12, 1, K)).astype(np.float32)
        bb = dev.upload(b)
        dev.mul_mat_f32(ab, bb, ob, K, N, 1, ne02, ne12, ne02 * N, 1, N)
        got = dev.download(ob, np.float32, (ne12, 1, N))
        emax, _ = npref.rel_err(got, oracle.mul_mat_f32(a_view, b))
        assert emax < 1e-5, rep
        dev.mul_mat_f32(ab, bb, ob, K, N, 1, ne02, ne12, ne02 * N, 1, N)
        assert np.array_equal(dev.download(ob, np.float32, (ne12, 1, N)), got)      # same bits every launch
