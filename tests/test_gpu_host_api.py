"""The galois op API (C++ host mirror over the C ABI) on the GPU, written the way the reference's own
tests are (src/cuda.rs:1701-1795, src/op.rs:3538-3650): build tensors, call galois_*, read back -- except
that these assert against the CPU oracle where the reference only prints."""
import numpy as np
import pytest

import oracle
from galois_amd import host_api as g
from tests import npref

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def gpu():
    return g.Device.gpu(0)


def test_cuda_matmul_gemv_and_prefill(gpu):
    rng = np.random.default_rng(1)
    k, n = 4096, 320
    w = oracle.quantize_q4_0((rng.standard_normal((n, k)) * 0.02).astype(np.float32))
    a = g.Tensor.from_raw(w, [k, n], g.Q4_0, gpu)
    for m, tol in ((1, 1e-4), (7, 2e-3), (130, 2e-3)):
        x = rng.standard_normal((m, k)).astype(np.float32)
        b = g.Tensor.from_raw(x, [k, m], g.F32, gpu)
        d = g.Tensor.zeros([n, m], g.F32, gpu)
        g.galois_matmul(a, b, d)
        got = d.to_cpu_tensor()
        assert got.shape == (m, n)
        emax, el2 = npref.rel_err(got.reshape(m, n), oracle.mul_mat_q4_0_f32(w, x))
        assert emax < tol and el2 < tol, (m, emax, el2)


@pytest.mark.parametrize("k,n,ne02,ne12", [(256, 48, 2, 4), (128, 40, 1, 11), (96, 8, 3, 3), (4096, 64, 4, 8)])
def test_cuda_matmul_batched_broadcast(gpu, k, n, ne02, ne12):
    """src0 [K, N, ne02] broadcast over src1 [K, 1, ne12] as in src/cuda.rs:1024-1034 (i02 = i12 / (ne12/ne02)):
    slices in one grouped launch per eight when the shape allows (K % 64 == 0), one launch per slice otherwise."""
    rng = np.random.default_rng(2 + k)
    w = oracle.quantize_q4_0((rng.standard_normal((ne02, n, k)) * 0.02).astype(np.float32))
    x = rng.standard_normal((ne12, 1, k)).astype(np.float32)
    a = g.Tensor.from_raw(w, [k, n, ne02], g.Q4_0, gpu)
    b = g.Tensor.from_raw(x, [k, 1, ne12], g.F32, gpu)
    d = g.Tensor.zeros([n, 1, ne12], g.F32, gpu)
    g.galois_matmul(a, b, d)
    got = d.to_cpu_tensor().reshape(ne12, n)
    for i in range(ne12):
        ref = oracle.mul_mat_q4_0_f32(w[i // (ne12 // ne02)], x[i, 0])
        emax, _ = npref.rel_err(got[i], ref)
        assert emax < 1e-4, i


def test_cuda_rmsnorm_rope_softmax(gpu):
    rng = np.random.default_rng(3)
    x = rng.standard_normal((5, 4096)).astype(np.float32)
    s, d = g.Tensor.from_raw(x, [4096, 5], g.F32, gpu), g.Tensor.zeros([4096, 5], g.F32, gpu)
    g.galois_rms_norm(s, d, 1e-6)
    emax, _ = npref.rel_err(d.to_cpu_tensor().reshape(5, 4096), oracle.rms_norm(x, 1e-6))
    assert emax < 1e-5

    t, h, hd = 6, 4, 128
    q = rng.standard_normal((t, h, hd)).astype(np.float32)
    pos = np.arange(3, 3 + t, dtype=np.int32)
    s0 = g.Tensor.from_raw(q, [hd, h, t], g.F32, gpu)
    s1 = g.Tensor.from_raw(pos, [t], g.I32, gpu)
    d = g.Tensor.zeros([hd, h, t], g.F32, gpu)
    g.galois_rope_custom({"n_dims": hd, "mode": 0, "freq_base": 10000.0, "freq_scale": 1.0}, s0, s1, d)
    ref = npref.rope(q, pos, h)
    assert np.max(np.abs(d.to_cpu_tensor().reshape(t, h, hd) - ref)) < 1e-4

    sc = (rng.standard_normal((3, 7, 64)) * 3).astype(np.float32)
    sc[:, :, 40:] = -np.inf
    s, d = g.Tensor.from_raw(sc, [64, 7, 3], g.F32, gpu), g.Tensor.zeros([64, 7, 3], g.F32, gpu)
    g.galois_soft_max(s, d)
    got = d.to_cpu_tensor().reshape(21, 64)
    emax, _ = npref.rel_err(got, oracle.soft_max(sc.reshape(21, 64)))
    assert emax < 1e-5 and np.all(got[:, 40:] == 0)


def test_view_is_pointer_arithmetic_in_elements(gpu):
    rng = np.random.default_rng(4)
    k, n = 128, 16
    w = oracle.quantize_q4_0((rng.standard_normal((n, k)) * 0.02).astype(np.float32))
    a = g.Tensor.from_raw(w, [k, n], g.Q4_0, gpu)
    tail = a.view(8 * k, [k, 8])  # rows 8..15: offset counted in weights, 18 bytes per 32 of them
    assert np.array_equal(tail.to_cpu_tensor(), w[8:].ravel())


def test_errors_instead_of_panics(gpu):
    cpu = g.Device.cpu()
    w = np.zeros(18 * 4, np.uint8)
    a = g.Tensor.from_raw(w, [128, 1], g.Q4_0, gpu)
    x = g.Tensor.zeros([128, 1], g.F32, gpu)
    y = g.Tensor.zeros([1, 1], g.F32, gpu)
    g.galois_matmul(a, x, y)
    with pytest.raises(g.GError) as e:   # the reference's (Cpu, Gpu, ..) arm is todo!()
        g.galois_matmul(g.Tensor.from_raw(w, [128, 1], g.Q4_0, cpu), x, y)
    assert e.value.kind == "Unimplemented"
    g.galois_matmul(x, x, y)             # f32 x f32 (todo!() in the reference, src/cuda.rs:867-879) is served here
    with pytest.raises(g.GError) as e:   # an i32 operand has no matmul arm (CudaMap2::map, src/cuda.rs:476-521)
        g.galois_matmul(g.Tensor.zeros([128, 1], g.I32, gpu), x, y)
    assert e.value.kind == "Unimplemented"
    with pytest.raises(g.GError) as e:   # assert!(ne0 == ne01) in the reference (src/op.rs:1422)
        g.galois_matmul(a, x, g.Tensor.zeros([2, 1], g.F32, gpu))
    assert e.value.kind == "ShapeError"
    with pytest.raises(g.GError) as e:   # NeoX mode: todo!() at src/cuda.rs:1336-1340
        g.galois_rope_custom({"n_dims": 128, "mode": 2}, x, g.Tensor.zeros([1], g.I32, gpu), x)
    assert e.value.kind == "Unimplemented"
    with pytest.raises(g.GError):        # ne0 not a multiple of the block size
        g.Tensor.zeros([48, 1], g.Q4_0, gpu)
    # the row kernels walk contiguous rows: a permuted view is refused, not read as if it were contiguous
    m = g.Tensor.zeros([64, 8], g.F32, gpu)
    mt = m.view_strided(0, [8, 64], [64, 1])     # the transpose
    out = g.Tensor.zeros([8, 64], g.F32, gpu)
    for call in (lambda: g.galois_rms_norm(mt, out, 1e-6), lambda: g.galois_soft_max(mt, out),
                 lambda: g.galois_soft_max(out, mt),
                 lambda: g.galois_rope_custom({"n_dims": 8, "mode": 0}, mt.view_strided(0, [8, 64, 1], [64, 1, 512]),
                                              g.Tensor.zeros([1], g.I32, gpu), out.view(0, [8, 64, 1]))):
        with pytest.raises(g.GError) as e:
            call()
        assert e.value.kind == "Unimplemented"
    with pytest.raises(g.GError) as e:
        g.Device.gpu(999)
    assert e.value.kind == "DeviceError"
