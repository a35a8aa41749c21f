"""Independent numpy restatements used to pin the C oracle (tests only).

Written from the published definitions, vectorised, sharing no code with
``oracle/galois_oracle.c``: a disagreement between the two is a bug in one of them.
"""
import numpy as np

QK = 32


def q4_0_unpack(q):
    """uint8 [..., nb*18] -> (d f32 [..., nb], nibbles int [..., nb, 32]) in weight order."""
    q = np.asarray(q, np.uint8)
    blk = q.reshape(q.shape[:-1] + (-1, 18))
    d = blk[..., :2].copy().view(np.float16)[..., 0].astype(np.float32)
    qs = blk[..., 2:].astype(np.int32)
    nib = np.concatenate([qs & 0xF, qs >> 4], axis=-1)  # weight j = low nibble j, j+16 = high nibble j
    return d, nib


def q4_0_dequant(q):
    d, nib = q4_0_unpack(q)
    w = (nib - 8).astype(np.float32) * d[..., None]
    return w.reshape(w.shape[:-2] + (-1,))


def q4_0_quantize(x):
    """Canonical ggml quantize_row_q4_0, vectorised (argmax of |x| picks the first maximum)."""
    x = np.asarray(x, np.float32)
    xb = x.reshape(x.shape[:-1] + (-1, QK))
    idx = np.argmax(np.abs(xb), axis=-1)
    mx = np.take_along_axis(xb, idx[..., None], axis=-1)[..., 0]
    d = (mx / np.float32(-8.0)).astype(np.float32)
    with np.errstate(divide="ignore"):
        inv = np.where(d != 0, np.float32(1.0) / d, np.float32(0.0)).astype(np.float32)
    t = (xb * inv[..., None]).astype(np.float32) + np.float32(8.5)
    qv = np.minimum(np.trunc(t.astype(np.float32)).astype(np.int32), 15).astype(np.uint8)
    qs = qv[..., :16] | (qv[..., 16:] << 4)
    dbytes = d.astype(np.float16)[..., None].view(np.uint8)
    out = np.concatenate([dbytes, qs], axis=-1)
    return out.reshape(x.shape[:-1] + (-1,))


def q8_0_quantize(x):
    """BlockQ8_0::from_f32: d = amax/127, q = round-half-away(x / d)."""
    x = np.asarray(x, np.float32)
    xb = x.reshape(x.shape[:-1] + (-1, QK))
    amax = np.max(np.abs(xb), axis=-1)
    d = (amax / np.float32(127.0)).astype(np.float32)
    with np.errstate(divide="ignore"):
        inv = np.where(d != 0, np.float32(1.0) / d, np.float32(0.0)).astype(np.float32)
    t = (xb * inv[..., None]).astype(np.float32)
    qv = (np.sign(t) * np.floor(np.abs(t) + np.float32(0.5))).astype(np.int8)
    dbytes = d.astype(np.float16)[..., None].view(np.uint8)
    out = np.concatenate([dbytes, qv.view(np.uint8)], axis=-1)
    return out.reshape(x.shape[:-1] + (-1,))


def q8_0_unpack(q):
    q = np.asarray(q, np.uint8)
    blk = q.reshape(q.shape[:-1] + (-1, 34))
    d = blk[..., :2].copy().view(np.float16)[..., 0].astype(np.float32)
    qs = blk[..., 2:].copy().view(np.int8).astype(np.int32)
    return d, qs


def rms_norm(x, eps, weight=None):
    x = np.asarray(x, np.float64)
    y = x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + np.float64(np.float32(eps)))
    if weight is not None:
        y = y * np.asarray(weight, np.float64)
    return y


def rope(x, pos, n_head, freq_base=10000.0, freq_scale=1.0, n_dims=None):
    """x [tokens, heads, head_dim] -> rotated, float64; adjacent-pair (non-NeoX) mode."""
    x = np.asarray(x, np.float64)
    t, h, hd = x.shape
    assert h == n_head
    n_dims = hd if n_dims is None else n_dims
    theta_scale = np.float64(np.float32(freq_base) ** np.float32(-2.0 / n_dims))
    i = np.arange(hd // 2, dtype=np.float64)
    theta = (np.asarray(pos, np.float64)[:, None] * np.float64(np.float32(freq_scale))) * theta_scale ** i
    c, s = np.cos(theta)[:, None, :], np.sin(theta)[:, None, :]
    x0, x1 = x[..., 0::2], x[..., 1::2]
    out = np.empty_like(x)
    out[..., 0::2] = x0 * c - x1 * s
    out[..., 1::2] = x0 * s + x1 * c
    return out


def rel_err(got, ref):
    """(max|d| / max|ref|, ||d||_2 / ||ref||_2) -- the two metrics the parity gates use."""
    got = np.asarray(got, np.float64)
    ref = np.asarray(ref, np.float64)
    d = got - ref
    den_max = max(np.max(np.abs(ref)), 1e-300)
    den_l2 = max(np.linalg.norm(ref.ravel()), 1e-300)
    return float(np.max(np.abs(d)) / den_max), float(np.linalg.norm(d.ravel()) / den_l2)


def rope_f32_angles(x, pos, freq_scale, p_delta_rows, theta_scale):
    """rope_f32 with the reference kernel's f32 angle (galois-kernels/src/rope.cu:16-20):
    theta = f32(f32(pos * freq_scale) * powf(theta_scale, col / 2)), then the rotation in f64.  What is left between
    this and an f32 kernel is the last bit of powf and of sin / cos, not the rounding of the angle itself."""
    x = np.asarray(x, np.float32)
    nrows, ncols = x.shape
    p0 = (np.asarray(pos, np.int64)[np.arange(nrows) // p_delta_rows].astype(np.float32) * np.float32(freq_scale))
    pw = np.power(np.float32(theta_scale), np.arange(ncols // 2, dtype=np.float32)).astype(np.float32)
    theta = (p0[:, None] * pw[None, :]).astype(np.float32).astype(np.float64)
    x0, x1 = x[:, 0::2].astype(np.float64), x[:, 1::2].astype(np.float64)
    out = np.empty(x.shape, np.float64)
    out[:, 0::2] = x0 * np.cos(theta) - x1 * np.sin(theta)
    out[:, 1::2] = x0 * np.sin(theta) + x1 * np.cos(theta)
    return out
