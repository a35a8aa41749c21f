"""The attention entry point that allocates nothing (galois_hip_attn_decode_f32_static: partial results in a static
device array) against galois_hip_attn_decode_f32, through the C ABI: bit-identical outputs and cache rows, on two
calls in a row, the second with a smaller input; then the limits."""
import numpy as np
import pytest

from galois_amd import GaloisHipError

pytestmark = pytest.mark.gpu


def _call(dev, fn, q, k, v, kc, vc, H, D, n_past):
    bufs = [dev.upload(a) for a in (q, k, v, kc, vc)]
    out = dev.alloc(H * D * 4 + 64)
    dev.upload(np.full(H * D + 16, 7.5, np.float32), out)
    pos = dev.upload(np.array([n_past], np.int32))
    ts = float(np.float32(10000.0) ** np.float32(-2.0 / D))
    fn(bufs[0], bufs[1], bufs[2], bufs[3], bufs[4], out, H, D, n_past, pos, 1.0, ts, float(1.0 / np.sqrt(D)))
    o = dev.download(out, np.float32, H * D + 16)
    assert np.all(o[H * D:] == 7.5), "wrote past the end of out"
    rows = (dev.download(bufs[3], np.float32, kc.shape)[n_past].copy(),
            dev.download(bufs[4], np.float32, vc.shape)[n_past].copy())
    for b in bufs + [out, pos]:
        dev.free(b)
    return o[:H * D], rows


def _case(seed, H, D, n_past):
    rng = np.random.default_rng(seed)
    E = H * D
    q, k, v = (rng.standard_normal(E).astype(np.float32) for _ in range(3))
    kc = rng.standard_normal((n_past + 1, E)).astype(np.float32)
    vc = rng.standard_normal((n_past + 1, E)).astype(np.float32)
    return q, k, v, kc, vc


def test_static_scratch_entry_point_matches_twice_in_a_row(dev):
    # the larger call first: what it leaves in the static block must not reach the smaller one
    for seed, (H, D, n_past) in enumerate(((32, 128, 2047), (8, 64, 300), (32, 128, 2047), (3, 128, 0))):
        c = _case(70 + seed, H, D, n_past)
        ref, ref_rows = _call(dev, dev.attn_decode_f32, *c, H, D, n_past)
        got, got_rows = _call(dev, dev.attn_decode_f32_static, *c, H, D, n_past)
        assert np.array_equal(got, ref), (H, D, n_past)
        assert np.array_equal(got_rows[0], ref_rows[0]) and np.array_equal(got_rows[1], ref_rows[1])


def test_static_scratch_limits(dev):
    buf = dev.alloc(4096)
    # 32 heads of 128: 62 splits (7936 positions) fit the static block, 63 do not; more than 1024 heads never do
    for H, D, n_past in ((32, 128, 62 * 128), (1025, 64, 200)):
        with pytest.raises(GaloisHipError) as ei:
            dev.attn_decode_f32_static(buf, buf, buf, buf, buf, buf, H, D, n_past, buf, 1.0, 1.0, 1.0)
        assert ei.value.status == -2
    dev.free(buf)
