"""ctypes loader for the CPU oracle (``oracle/galois_oracle.c``).

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, ``__graft_entry__.smoke()`` and
the ``cpu_baseline`` leg of ``bench.py``.  The product package never imports it.
All arrays are C-contiguous numpy arrays; Q4_0 / Q8_0 data are ``uint8`` arrays
holding the reference's block bytes (18 B and 34 B per 32 values).
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
# GALOIS_ORACLE_LIB: another build of the same library (`make sanitize`: address + undefined-behaviour sanitizers)
_SO = os.environ.get("GALOIS_ORACLE_LIB") or os.path.join(_HERE, "libgalois_oracle.so")

QK = 32
Q4_0_BYTES = 18
Q8_0_BYTES = 34


def build(force=False):
    """Compile the oracle with the committed Makefile (gcc, a few seconds)."""
    if force and os.path.exists(_SO):
        os.remove(_SO)
    subprocess.check_call(["make", "-s", "-C", _HERE])
    return _SO


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        L = C.CDLL(_SO)
        f32p, u8p, u16p, i32p = (C.POINTER(C.c_float), C.POINTER(C.c_uint8),
                                 C.POINTER(C.c_uint16), C.POINTER(C.c_int32))
        i64 = C.c_int64
        sig = {
            "orc_f16_to_f32_row": (None, [u16p, f32p, i64]),
            "orc_f32_to_f16_row": (None, [f32p, u16p, i64]),
            "orc_quantize_row_q4_0": (None, [f32p, u8p, i64]),
            "orc_dequantize_row_q4_0": (None, [u8p, f32p, i64]),
            "orc_quantize_row_q8_0": (None, [f32p, u8p, i64]),
            "orc_vec_dot_q4_0_q8_0_scalar": (C.c_float, [i64, u8p, u8p]),
            "orc_vec_dot_q4_0_q8_0_avx2": (C.c_float, [i64, u8p, u8p]),
            "orc_mul_mat_q4_0_f32": (None, [u8p, f32p, f32p, i64, i64, i64, C.c_int]),
            "orc_cpu_mul_mat_q4_0_f32": (None, [u8p, f32p, f32p, i64, i64, i64, C.c_int]),
            "orc_rms_norm_f32": (None, [f32p, f32p, i64, i64, C.c_float]),
            "orc_mul_f32": (None, [f32p, f32p, f32p, i64, i64]),
            "orc_add_f32": (None, [f32p, f32p, f32p, i64, i64]),
            "orc_scale_f32": (None, [f32p, f32p, C.c_float, i64]),
            "orc_silu_f32": (None, [f32p, f32p, i64]),
            "orc_rope_f32": (None, [f32p, f32p, i64, i64, i32p, C.c_float, i64, C.c_float]),
            "orc_soft_max_f32": (None, [f32p, f32p, i64, i64]),
            "orc_soft_max_causal_f32": (None, [f32p, f32p, i64, i64, i64, i64]),
            "orc_mul_mat_f32": (None, [f32p, f32p, f32p, i64, i64, i64, i64, i64, i64, i64, i64]),
            "orc_cpy_f32": (None, [C.c_void_p, C.c_void_p, C.c_int] + [i64] * 11),
            "orc_get_rows_q4_0": (None, [u8p, i32p, f32p, i64, i64]),
            "orc_sizeof_block_q4_0": (C.c_int, []),
            "orc_sizeof_block_q8_0": (C.c_int, []),
            "orc_have_avx2": (C.c_int, []),
        }
        for name, (res, args) in sig.items():
            fn = getattr(L, name)
            fn.restype, fn.argtypes = res, args
        _lib = L
    return _lib


def _p(a, ct):
    return a.ctypes.data_as(C.POINTER(ct))


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _u8(a):
    a = np.ascontiguousarray(a)
    assert a.dtype == np.uint8
    return a


def f16_to_f32(h):
    h = np.ascontiguousarray(h, dtype=np.uint16)
    out = np.empty(h.shape, np.float32)
    lib().orc_f16_to_f32_row(_p(h, C.c_uint16), _p(out, C.c_float), h.size)
    return out


def f32_to_f16(f):
    f = _f32(f)
    out = np.empty(f.shape, np.uint16)
    lib().orc_f32_to_f16_row(_p(f, C.c_float), _p(out, C.c_uint16), f.size)
    return out


def quantize_q4_0(x):
    """f32 [..., K] -> uint8 [..., K/32*18] (blocks along the last axis)."""
    x = _f32(x)
    k = x.shape[-1]
    assert k % QK == 0
    out = np.empty(x.shape[:-1] + (k // QK * Q4_0_BYTES,), np.uint8)
    lib().orc_quantize_row_q4_0(_p(x, C.c_float), _p(out, C.c_uint8), x.size)
    return out


def dequantize_q4_0(q):
    q = _u8(q)
    nb = q.shape[-1] // Q4_0_BYTES
    assert nb * Q4_0_BYTES == q.shape[-1]
    out = np.empty(q.shape[:-1] + (nb * QK,), np.float32)
    lib().orc_dequantize_row_q4_0(_p(q, C.c_uint8), _p(out, C.c_float), out.size)
    return out


def quantize_q8_0(x):
    x = _f32(x)
    k = x.shape[-1]
    assert k % QK == 0
    out = np.empty(x.shape[:-1] + (k // QK * Q8_0_BYTES,), np.uint8)
    lib().orc_quantize_row_q8_0(_p(x, C.c_float), _p(out, C.c_uint8), x.size)
    return out


def vec_dot_q4_0_q8_0(wq, xq, kind="avx2"):
    wq, xq = _u8(wq), _u8(xq)
    n = wq.size // Q4_0_BYTES * QK
    assert xq.size // Q8_0_BYTES * QK == n
    fn = lib().orc_vec_dot_q4_0_q8_0_avx2 if kind == "avx2" else lib().orc_vec_dot_q4_0_q8_0_scalar
    return float(fn(n, _p(wq, C.c_uint8), _p(xq, C.c_uint8)))


def mul_mat_q4_0_f32(wq, x, nthreads=8):
    """Parity oracle: dequant-then-dot in f64.  wq uint8 [N, K/32*18], x f32 [M, K] or [K]."""
    wq = _u8(wq)
    x = _f32(x)
    vec = x.ndim == 1
    x2 = x.reshape(1, -1) if vec else x
    n, k, m = wq.shape[0], x2.shape[1], x2.shape[0]
    assert wq.shape[1] == k // QK * Q4_0_BYTES
    y = np.empty((m, n), np.float32)
    lib().orc_mul_mat_q4_0_f32(_p(wq, C.c_uint8), _p(x2, C.c_float), _p(y, C.c_float), k, n, m, nthreads)
    return y[0] if vec else y


def cpu_mul_mat_q4_0_f32(wq, x, nth=4):
    """The reference CPU op (Q8_0 activations + integer dot): the timed baseline."""
    wq = _u8(wq)
    x = _f32(x)
    vec = x.ndim == 1
    x2 = x.reshape(1, -1) if vec else x
    n, k, m = wq.shape[0], x2.shape[1], x2.shape[0]
    y = np.empty((m, n), np.float32)
    lib().orc_cpu_mul_mat_q4_0_f32(_p(wq, C.c_uint8), _p(x2, C.c_float), _p(y, C.c_float), k, n, m, nth)
    return y[0] if vec else y


def rms_norm(x, eps):
    x = _f32(x)
    y = np.empty_like(x)
    lib().orc_rms_norm_f32(_p(x, C.c_float), _p(y, C.c_float), x.shape[-1], x.size // x.shape[-1], eps)
    return y


def _bcast(fn, x, yv):
    x, yv = _f32(x), _f32(yv)
    out = np.empty_like(x)
    fn(_p(x, C.c_float), _p(yv, C.c_float), _p(out, C.c_float), x.size, yv.size)
    return out


def mul(x, yv):
    return _bcast(lib().orc_mul_f32, x, yv)


def add(x, yv):
    return _bcast(lib().orc_add_f32, x, yv)


def scale(x, s):
    x = _f32(x)
    out = np.empty_like(x)
    lib().orc_scale_f32(_p(x, C.c_float), _p(out, C.c_float), s, x.size)
    return out


def silu(x):
    x = _f32(x)
    out = np.empty_like(x)
    lib().orc_silu_f32(_p(x, C.c_float), _p(out, C.c_float), x.size)
    return out


def rope(x, pos, freq_scale, p_delta_rows, theta_scale):
    """x f32 [nrows, ncols] (rows = tokens*heads, token-major), pos int32 [tokens]."""
    x = _f32(x)
    pos = np.ascontiguousarray(pos, dtype=np.int32)
    ncols = x.shape[-1]
    nrows = x.size // ncols
    out = np.empty_like(x)
    lib().orc_rope_f32(_p(x, C.c_float), _p(out, C.c_float), ncols, nrows, _p(pos, C.c_int32),
                       freq_scale, p_delta_rows, theta_scale)
    return out


def soft_max(x):
    x = _f32(x)
    out = np.empty_like(x)
    lib().orc_soft_max_f32(_p(x, C.c_float), _p(out, C.c_float), x.shape[-1], x.size // x.shape[-1])
    return out


def soft_max_causal(x, rows_per_head, n_past=0):
    x = _f32(x)
    out = np.empty_like(x)
    lib().orc_soft_max_causal_f32(_p(x, C.c_float), _p(out, C.c_float), x.shape[-1], rows_per_head,
                                  x.size // x.shape[-1], n_past)
    return out


def mul_mat_f32(a, b):
    """a f32 [ne02, N, K] (any strides), b f32 [ne12, M, K] contiguous -> [ne12, M, N]."""
    assert a.dtype == np.float32 and a.ndim == 3
    b = _f32(b)
    ne02, n, k = a.shape
    ne12, m, kb = b.shape
    assert kb == k and ne12 % ne02 == 0
    s2, s1, s0 = (s // 4 for s in a.strides)
    out = np.empty((ne12, m, n), np.float32)
    lib().orc_mul_mat_f32(_p(a, C.c_float), _p(b, C.c_float), _p(out, C.c_float), k, n, m, ne02, ne12,
                          s0, s1, s2)
    return out


def cpy_f32(src, dst, ne, ne00, ne01, nb0, ne10, ne11, nb1):
    """Strided copy (byte strides nb0 = (nb00, nb01, nb02), nb1 likewise) into a float32 or float16 array."""
    assert src.dtype == np.float32 and dst.dtype in (np.float32, np.float16)
    lib().orc_cpy_f32(src.ctypes.data_as(C.c_void_p), dst.ctypes.data_as(C.c_void_p), int(dst.dtype == np.float16),
                      ne, ne00, ne01, nb0[0], nb0[1], nb0[2], ne10, ne11, nb1[0], nb1[1], nb1[2])
    return dst


def get_rows_q4_0(table, ids):
    table = _u8(table)
    ids = np.ascontiguousarray(ids, np.int32)
    ncols = table.shape[1] // Q4_0_BYTES * QK
    out = np.empty((ids.size, ncols), np.float32)
    lib().orc_get_rows_q4_0(_p(table, C.c_uint8), _p(ids, C.c_int32), _p(out, C.c_float), ncols, ids.size)
    return out
