"""GPU parity of the Q4_0 quantizer / dequantizer: bytes identical to the CPU oracle."""
import json
import os

import numpy as np
import pytest

import oracle

pytestmark = pytest.mark.gpu
KAT = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "kat.json")))


def _quant(dev, x):
    x = np.ascontiguousarray(x, np.float32)
    xb = dev.upload(x)
    nbytes = x.size // 32 * 18
    yb = dev.alloc(nbytes + 64)
    dev.upload(np.full(nbytes + 64, 0xAB, np.uint8), yb)
    dev.quantize_row_q4_0(xb, yb, x.size)
    out = dev.download(yb, np.uint8, nbytes + 64)
    assert np.all(out[nbytes:] == 0xAB)
    dev.free(xb), dev.free(yb)
    return out[:nbytes]


@pytest.mark.parametrize("name", sorted(KAT["quantize_q4_0"]))
def test_quantize_kat(dev, name):
    c = KAT["quantize_q4_0"][name]
    assert _quant(dev, np.array(c["x"], np.float32)).tolist() == c["block"], c["why"]


def test_quantize_bytes_identical_to_oracle(dev):
    rng = np.random.default_rng(21)
    for scale in (0.02, 1.0, 1e-7, 3e4):
        x = (rng.standard_normal((257, 4096)) * scale).astype(np.float32)
        assert np.array_equal(_quant(dev, x), oracle.quantize_q4_0(x).ravel()), scale
    x = rng.integers(-8, 9, size=(4096, 64)).astype(np.float32)  # ties and exact .5 boundaries
    assert np.array_equal(_quant(dev, x), oracle.quantize_q4_0(x).ravel())
    assert np.array_equal(_quant(dev, x), _quant(dev, x.copy()))  # determinism


def test_dequantize_exact_and_round_trip(dev):
    rng = np.random.default_rng(22)
    x = (rng.standard_normal((64, 4096)) * 0.02).astype(np.float32)
    q = oracle.quantize_q4_0(x)
    qb = dev.upload(q)
    yb = dev.alloc(x.nbytes)
    dev.dequantize_row_q4_0(qb, yb, x.size)
    w = dev.download(yb, np.float32, x.shape)
    assert np.array_equal(w, oracle.dequantize_q4_0(q))
    # encode -> decode -> encode is idempotent on the nibbles
    q2 = _quant(dev, w).reshape(q.shape)
    w2 = oracle.dequantize_q4_0(q2)
    assert np.allclose(w2, w, rtol=0, atol=np.max(np.abs(w)) * 2.0 ** -9)
    dev.free(qb), dev.free(yb)
