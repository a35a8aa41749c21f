"""GPU parity of the M > 1 attention products (scores = K^T q and out = V p over many positions at once) against
the oracle's f64 contraction: the f32 matrix-core kernel multiplies and accumulates in f32 and widens an f16 operand
exactly, so the bar is the 1e-5 of the one-row kernels, for f32 and f16 caches, both orientations of the cache view,
ragged sizes, and a broadcast over the batch.  One case takes another kernel: an f16 cache read along K in rows of a
multiple of 32 goes to the f16 matrix-core kernel, which rounds b to f16 as the reference's convert_fp32_to_fp16 does
(bar 2e-3, as in tests/test_gpu_matmul_f16.py).  (The reference routes these to cuBLAS, src/cuda.rs:698-782, 881-992,
and holds no expected values for them.)"""
import numpy as np
import pytest

import oracle
from tests import npref

pytestmark = pytest.mark.gpu


def _mm(dev, f16):
    return dev.mul_mat_f16_f32 if f16 else dev.mul_mat_f32


@pytest.mark.parametrize("L,H,D,M,f16", [(512, 32, 128, 512, False), (300, 4, 128, 70, False), (77, 3, 64, 16, False),
                                         (512, 8, 128, 512, True), (333, 2, 64, 129, True), (40, 1, 80, 17, False)])
def test_prefill_attention_products(dev, L, H, D, M, f16):
    rng = np.random.default_rng(L + H + M)
    ct = np.float16 if f16 else np.float32
    kc = rng.standard_normal((L, H * D)).astype(ct)
    vc = rng.standard_normal((L, H * D)).astype(ct)
    q = rng.standard_normal((H, M, D)).astype(np.float32)
    kb, vb, qb = dev.upload(kc), dev.upload(vc), dev.upload(q)
    sb, ob = dev.alloc(H * M * L * 4 + 64), dev.alloc(H * M * D * 4 + 64)
    dev.upload(np.full(H * M * L + 16, 7.5, np.float32), sb)
    dev.upload(np.full(H * M * D + 16, 7.5, np.float32), ob)
    k32, v32 = kc.astype(np.float32), vc.astype(np.float32)
    kview = np.lib.stride_tricks.as_strided(k32, (H, L, D), (D * 4, H * D * 4, 4))
    vview = np.lib.stride_tricks.as_strided(v32, (H, D, L), (D * 4, 4, H * D * 4))
    # scores[h][m][l] = sum_d K[l][h*D+d] q[h][m][d]: a = view [ne0 = D, ne1 = L, ne2 = H], strides (1, H*D, D)
    _mm(dev, f16)(kb, qb, sb, D, L, M, H, H, 1, H * D, D)
    got = dev.download(sb, np.float32, H * M * L + 16)
    assert np.all(got[H * M * L:] == 7.5), "wrote past the end of dst"
    ref = oracle.mul_mat_f32(kview, q)
    emax, el2 = npref.rel_err(got[:H * M * L].reshape(H, M, L), ref)
    tol = 2e-3 if f16 and D % 32 == 0 else 1e-5
    assert emax < tol and el2 < tol, (emax, el2)
    # out[h][m][d] = sum_l V[l][h*D+d] p[h][m][l]: a = view [ne0 = L, ne1 = D, ne2 = H], strides (H*D, 1, D)
    p = oracle.soft_max((ref.reshape(H * M, L) / np.sqrt(D)).astype(np.float32)).reshape(H, M, L)
    pb = dev.upload(p)
    _mm(dev, f16)(vb, pb, ob, L, D, M, H, H, H * D, 1, D)
    got = dev.download(ob, np.float32, H * M * D + 16)
    assert np.all(got[H * M * D:] == 7.5), "wrote past the end of dst"
    emax, el2 = npref.rel_err(got[:H * M * D].reshape(H, M, D), oracle.mul_mat_f32(vview, p))
    assert emax < 1e-5 and el2 < 1e-5, (emax, el2)
    # unit rows of b select exact rows of the cache
    e = np.zeros((H, M, D), np.float32)
    e[:, :, D // 3] = 1.0
    dev.upload(e, qb)
    _mm(dev, f16)(kb, qb, sb, D, L, M, H, H, 1, H * D, D)
    got = dev.download(sb, np.float32, (H, M, L))
    for h in range(H):
        assert np.array_equal(got[h], np.tile(k32[:, h * D + D // 3], (M, 1)))
    for b in (kb, vb, qb, sb, ob, pb):
        dev.free(b)


def test_many_rows_with_a_broadcast_over_the_batch(dev):
    rng = np.random.default_rng(3)
    K, N, M, ne02, ne12 = 200, 130, 33, 2, 6
    a = rng.standard_normal((ne02, N, K)).astype(np.float32)
    b = rng.standard_normal((ne12, M, K)).astype(np.float32)
    ab, bb, ob = dev.upload(a), dev.upload(b), dev.alloc(ne12 * M * N * 4)
    dev.mul_mat_f32(ab, bb, ob, K, N, M, ne02, ne12, 1, K, N * K)
    emax, el2 = npref.rel_err(dev.download(ob, np.float32, (ne12, M, N)), oracle.mul_mat_f32(a, b))
    assert emax < 1e-5 and el2 < 1e-5
    for x in (ab, bb, ob):
        dev.free(x)
