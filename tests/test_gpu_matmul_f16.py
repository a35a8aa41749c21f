"""GPU parity of the (F16, F32) -> F32 matmul arm (galois_hip_mul_mat_f16_f32 and galois_matmul with an F16 src0)
against the oracle: the f16 operand widened exactly, contraction in f64.

The reference serves this arm with cuBLAS gemm_ex on f16 operands, f16 accumulation and an f16 result
(src/cuda.rs:881-992, 698-757); no test of the reference pins its output.  Bars here: decode shapes (M = 1, the a
operand widened, sums in f32) 1e-5; M > 1 on the matrix cores (b rounded to f16 like the reference's
convert_fp32_to_fp16, sums in f32) 2e-3, the prefill bar.
"""
import numpy as np
import pytest

import oracle
from galois_amd import host_api as g
from tests import npref

pytestmark = pytest.mark.gpu


def _views(c16, H, L, D):
    """K^T-style view [H, L, D] and V-style view [H, D, L] of a cache [L][H * D], as f32 arrays for the oracle."""
    c32 = c16.astype(np.float32)
    return (np.lib.stride_tricks.as_strided(c32, (H, L, D), (D * 4, H * D * 4, 4)),
            np.lib.stride_tricks.as_strided(c32, (H, D, L), (D * 4, 4, H * D * 4)))


@pytest.mark.parametrize("L,H,D", [(300, 4, 128), (2048, 32, 128), (77, 3, 64)])
def test_attention_products_over_an_f16_kv_cache(dev, L, H, D):
    rng = np.random.default_rng(L + H)
    kc = rng.standard_normal((L, H * D)).astype(np.float16)
    vc = rng.standard_normal((L, H * D)).astype(np.float16)
    q = rng.standard_normal((H, 1, D)).astype(np.float32)
    kb, vb, qb = dev.upload(kc), dev.upload(vc), dev.upload(q)
    sb, ob = dev.alloc(H * L * 4), dev.alloc(H * D * 4)
    kview, _ = _views(kc, H, L, D)
    _, vview = _views(vc, H, L, D)
    dev.mul_mat_f16_f32(kb, qb, sb, D, L, 1, H, H, 1, H * D, D)             # scores = K^T q
    ref = oracle.mul_mat_f32(kview, q)
    emax, el2 = npref.rel_err(dev.download(sb, np.float32, (H, 1, L)), ref)
    assert emax < 1e-5 and el2 < 1e-5
    p = oracle.soft_max((ref.reshape(H, L) / np.sqrt(D)).astype(np.float32)).reshape(H, 1, L)
    pb = dev.upload(p)
    dev.mul_mat_f16_f32(vb, pb, ob, L, D, 1, H, H, H * D, 1, D)             # out = V p
    emax, el2 = npref.rel_err(dev.download(ob, np.float32, (H, 1, D)), oracle.mul_mat_f32(vview, p))
    assert emax < 1e-5 and el2 < 1e-5
    for b in (kb, vb, qb, sb, ob, pb):
        dev.free(b)


@pytest.mark.parametrize("K,N,M,ne02,ne12", [(4096, 4096, 64, 1, 1), (128, 2048, 512, 4, 4), (96, 200, 70, 1, 3),
                                             (32, 1, 2, 2, 4), (4096, 300, 129, 1, 1)])
def test_f16_weights_on_the_matrix_cores(dev, K, N, M, ne02, ne12):
    rng = np.random.default_rng(K + N + M)
    a = (rng.standard_normal((ne02, N, K)) * 0.05).astype(np.float16)
    b = rng.standard_normal((ne12, M, K)).astype(np.float32)
    ab, bb, ob = dev.upload(a), dev.upload(b), dev.alloc(ne12 * M * N * 4 + 64)
    dev.upload(np.full(ne12 * M * N + 16, 7.5, np.float32), ob)
    dev.mul_mat_f16_f32(ab, bb, ob, K, N, M, ne02, ne12, 1, K, N * K)
    got = dev.download(ob, np.float32, ne12 * M * N + 16)
    assert np.all(got[ne12 * M * N:] == 7.5), "wrote past the end of dst"
    ref = oracle.mul_mat_f32(a.astype(np.float32), b)
    emax, el2 = npref.rel_err(got[:ne12 * M * N].reshape(ne12, M, N), ref)
    assert emax < 2e-3 and el2 < 2e-3, (emax, el2)
    # unit rows of b select exact rows of a: no rounding anywhere
    e = np.zeros((ne12, M, K), np.float32)
    e[:, :, K // 2] = 1.0
    dev.upload(e, bb)
    dev.mul_mat_f16_f32(ab, bb, ob, K, N, M, ne02, ne12, 1, K, N * K)
    got = dev.download(ob, np.float32, (ne12, M, N))
    for i2 in range(ne12):
        assert np.array_equal(got[i2], np.tile(a[i2 // (ne12 // ne02), :, K // 2].astype(np.float32), (M, 1)))
    for x in (ab, bb, ob):
        dev.free(x)


def test_one_row_and_many_rows_of_the_same_operands_agree_within_the_stated_rounding(dev):
    """The arm rounds b to f16 only where it runs on the matrix cores (M > 1, rows of a contiguous along K,
    K % 32 == 0); one row of activations (decode) keeps b in f32.  The same row multiplied both ways therefore
    differs by b's rounding and by nothing else: at most 2^-11 relative per element of b, i.e. within
    2^-11 * sum |a| |b| element by element (1e-3 of the largest result on these operands); with activations that f16
    holds exactly the two paths agree to the order of their f32 sums."""
    rng = np.random.default_rng(17)
    K, N, M = 4096, 512, 33
    a = (rng.standard_normal((1, N, K)) * 0.05).astype(np.float16)
    b = rng.standard_normal((1, M, K)).astype(np.float32)
    ab, ob = dev.upload(a), dev.alloc(M * N * 4)

    def both(bm):
        bb = dev.upload(bm)
        dev.mul_mat_f16_f32(ab, bb, ob, K, N, M, 1, 1, 1, K, N * K)            # M rows: matrix cores, b rounded to f16
        many = dev.download(ob, np.float32, (M, N))
        one = np.empty_like(many)
        for r in range(M):                                                      # row by row: b stays f32
            dev.mul_mat_f16_f32(ab, bb.view(r * K * 4), ob, K, N, 1, 1, 1, 1, K, N * K)
            one[r] = dev.download(ob, np.float32, N)
        dev.free(bb)
        return many, one

    many, one = both(b)
    bound = 2.0 ** -11 * (np.abs(b[0]).astype(np.float64) @ np.abs(a[0].astype(np.float64)).T)
    assert np.all(np.abs(many.astype(np.float64) - one) <= bound + 1e-5 * np.max(np.abs(one)))
    emax, el2 = npref.rel_err(many, one)
    assert emax < 1e-3 and el2 < 1e-3, (emax, el2)
    many, one = both(b.astype(np.float16).astype(np.float32))                   # nothing left to round
    emax, el2 = npref.rel_err(many, one)
    assert emax < 1e-5 and el2 < 1e-5, (emax, el2)
    for x in (ab, ob):
        dev.free(x)


def test_operands_the_matrix_core_kernel_does_not_take(dev):
    """K not a multiple of 32, or rows of a that are not 16-byte aligned: the generic kernels, exact widening."""
    rng = np.random.default_rng(5)
    K, N, M = 40, 9, 3
    a = rng.standard_normal((1, N, K)).astype(np.float16)
    b = rng.standard_normal((1, M, K)).astype(np.float32)
    ab, bb, ob = dev.upload(a), dev.upload(b), dev.alloc(M * N * 4)
    dev.mul_mat_f16_f32(ab, bb, ob, K, N, M, 1, 1, 1, K, N * K)
    emax, _ = npref.rel_err(dev.download(ob, np.float32, (1, M, N)), oracle.mul_mat_f32(a.astype(np.float32), b))
    assert emax < 1e-5
    for x in (ab, bb, ob):
        dev.free(x)


def test_galois_matmul_with_an_f16_src0():
    gpu = g.Device.gpu(0)
    rng = np.random.default_rng(6)
    K, N, M = 256, 48, 5
    w = (rng.standard_normal((N, K)) * 0.1).astype(np.float16)
    x = rng.standard_normal((M, K)).astype(np.float32)
    a = g.Tensor.from_raw(w, [K, N], g.F16, gpu)
    b = g.Tensor.from_raw(x, [K, M], g.F32, gpu)
    y = g.Tensor.zeros([N, M], g.F32, gpu)
    g.galois_matmul(a, b, y)
    ref = oracle.mul_mat_f32(w.astype(np.float32)[None], x[None])[0]
    emax, el2 = npref.rel_err(y.to_cpu_tensor(), ref)
    assert emax < 2e-3 and el2 < 2e-3
    # a decode-shaped product through the op API: one row of activations
    y1 = g.Tensor.zeros([N, 1], g.F32, gpu)
    g.galois_matmul(a, g.Tensor.from_raw(x[:1], [K, 1], g.F32, gpu), y1)
    emax, _ = npref.rel_err(y1.to_cpu_tensor(), ref[:1])
    assert emax < 1e-5
