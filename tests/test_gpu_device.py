"""GPU checks of the device / stream / buffer layer of the C ABI."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def test_device_info_is_gfx950(dev):
    info = dev.info()
    print(info)
    assert info["arch"].startswith("gfx950")
    assert info["n_cu"] > 0
    assert dev.n_kernels == 16


def test_alloc_is_zeroed_and_copies_round_trip(dev):
    rng = np.random.default_rng(0)
    buf = dev.alloc(1 << 20)
    assert np.all(dev.download(buf, np.uint8, 1 << 20) == 0)
    a = rng.integers(0, 256, 1 << 20, dtype=np.uint8)
    dev.upload(a, buf)
    assert np.array_equal(dev.download(buf, np.uint8, 1 << 20), a)
    # views are pointer arithmetic in bytes (18 per Q4_0 block)
    assert np.array_equal(dev.download(buf.view(18 * 5), np.uint8, 36), a[90:126])
    dst = dev.alloc(1 << 20)
    dev.copy_d2d(dst, buf, 1 << 20)
    assert np.array_equal(dev.download(dst, np.uint8, 1 << 20), a)
    # 2-D copy: 16 rows of 100 bytes from pitch 128 to pitch 256
    dst2 = dev.alloc(16 * 256)
    dev.copy_d2d_2d(dst2, 256, buf, 128, 100, 16)
    got = dev.download(dst2, np.uint8, (16, 256))
    assert np.array_equal(got[:, :100], a[:16 * 128].reshape(16, 128)[:, :100])
    assert np.all(got[:, 100:] == 0)
    for b in (buf, dst, dst2):
        dev.free(b)


def test_empty_alloc_and_bad_ordinal(dev):
    import galois_amd
    b = dev.alloc(0)
    assert b.ptr == 0
    with pytest.raises(galois_amd.GaloisHipError) as ei:
        galois_amd.Device(1000)
    assert ei.value.status == -4


def test_events_time_the_stream(dev):
    e0, e1 = dev.event(), dev.event()
    buf = dev.alloc(64 << 20)
    dst = dev.alloc(64 << 20)
    dev.record(e0)
    for _ in range(4):
        dev.copy_d2d(dst, buf, 64 << 20)
    dev.record(e1)
    ms = dev.elapsed_ms(e0, e1)
    assert 0 < ms < 1000
    dev.event_destroy(e0)
    dev.event_destroy(e1)
    dev.free(buf)
    dev.free(dst)
