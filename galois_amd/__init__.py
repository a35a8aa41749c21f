"""galois_amd -- MI355X (gfx950) backend for galois's Q4_0 quantized-matmul path.

The product is ``libgalois_hip.so`` (hand-written HIP kernels behind the C ABI of
``include/galois_hip.h``).  This package is the thin Python face of that ABI used by
the tests and the benchmark: device buffers, copies, events and one method per entry
point, argument for argument.  There is no CPU fallback: importing works anywhere,
but creating a :class:`Device` without the built library or without a gfx950 GPU
raises.
"""
import ctypes as C

import numpy as np

from . import _abi

__all__ = ["Device", "DeviceBuffer", "GaloisHipError", "Q4_0_BLOCK_BYTES", "QK4_0"]

QK4_0 = 32
Q4_0_BLOCK_BYTES = 18


class GaloisHipError(RuntimeError):
    def __init__(self, status, text):
        super().__init__("galois_hip status %d: %s" % (status, text))
        self.status = status


class DeviceBuffer:
    """Owning handle of device memory (the reference's CudaSlice<T>); ``ptr`` is a raw address."""

    def __init__(self, dev, ptr, nbytes, owner=True):
        self.dev, self.ptr, self.nbytes, self._owner = dev, ptr, nbytes, owner

    def view(self, byte_offset, nbytes=None):
        """Sub-view by pointer arithmetic (``.slice(offset..)`` in the reference, src/cuda.rs:54-73)."""
        assert 0 <= byte_offset <= self.nbytes
        nbytes = self.nbytes - byte_offset if nbytes is None else nbytes
        assert byte_offset + nbytes <= self.nbytes
        return DeviceBuffer(self.dev, self.ptr + byte_offset, nbytes, owner=False)

    def free(self):
        if self._owner and self.ptr:
            self.dev._check(self.dev._lib.galois_hip_free(self.dev._ctx, self.ptr))
            self.ptr = 0

    def __int__(self):
        return self.ptr


def _ptr(b):
    if b is None:
        return None
    return C.c_void_p(b.ptr if isinstance(b, DeviceBuffer) else int(b))


class Device:
    """One device ordinal + one stream (``CudaDevice::new``, src/cuda.rs:221-229)."""

    def __init__(self, ordinal=0):
        self._lib = _abi.load()
        ctx = C.c_void_p()
        st = self._lib.galois_hip_create(ordinal, C.byref(ctx))
        if st != 0:
            raise GaloisHipError(st, self._lib.galois_hip_status_string(st).decode())
        self._ctx = ctx
        self._bufs = []
        n = C.c_int32()
        self._check(self._lib.galois_hip_init_functions(self._ctx, _abi.ABI_VERSION, C.byref(n)))
        self.n_kernels = n.value

    # -- plumbing ---------------------------------------------------------------
    def _check(self, st):
        if st != 0:
            raise GaloisHipError(st, self._lib.galois_hip_last_error(self._ctx).decode()
                                 or self._lib.galois_hip_status_string(st).decode())

    def close(self):
        if self._ctx:
            for b in self._bufs:
                b.free()
            self._bufs = []
            self._lib.galois_hip_destroy(self._ctx)
            self._ctx = None

    OPT_GEMV_F32_ARITHMETIC, OPT_WAIT_SPIN_LIMIT, OPT_WAIT_TARGET_BIAS = 1, 2, 3

    def set_option(self, option, value):
        self._check(self._lib.galois_hip_set_option(self._ctx, option, value))

    def info(self):
        name, arch = C.create_string_buffer(256), C.create_string_buffer(256)
        ncu, clk, mclk, mem = C.c_int32(), C.c_int32(), C.c_int32(), C.c_int64()
        self._check(self._lib.galois_hip_device_info(self._ctx, name, 256, arch, 256, C.byref(ncu), C.byref(clk),
                                                     C.byref(mclk), C.byref(mem)))
        return {"name": name.value.decode(), "arch": arch.value.decode(), "n_cu": ncu.value,
                "clock_khz": clk.value, "mem_clock_khz": mclk.value, "mem_bytes": mem.value}

    def alloc(self, nbytes):
        p = C.c_void_p()
        self._check(self._lib.galois_hip_alloc_zeros(self._ctx, nbytes, C.byref(p)))
        b = DeviceBuffer(self, p.value or 0, nbytes)
        self._bufs.append(b)
        return b

    def free(self, buf):
        buf.free()
        self._bufs = [b for b in self._bufs if b is not buf]

    def upload(self, arr, buf=None):
        arr = np.ascontiguousarray(arr)
        if buf is None:
            buf = self.alloc(arr.nbytes)
        assert arr.nbytes <= buf.nbytes
        self._check(self._lib.galois_hip_htod_sync_copy(self._ctx, _ptr(buf), arr.ctypes.data_as(C.c_void_p),
                                                        arr.nbytes))
        return buf

    def download(self, buf, dtype, shape):
        out = np.empty(shape, dtype)
        assert out.nbytes <= buf.nbytes
        self._check(self._lib.galois_hip_dtoh_sync_copy(self._ctx, out.ctypes.data_as(C.c_void_p), _ptr(buf),
                                                        out.nbytes))
        return out

    def copy_d2d(self, dst, src, nbytes):
        self._check(self._lib.galois_hip_dtod_copy(self._ctx, _ptr(dst), _ptr(src), nbytes))

    def copy_d2d_2d(self, dst, dpitch, src, spitch, width, height):
        self._check(self._lib.galois_hip_dtod_copy_2d(self._ctx, _ptr(dst), dpitch, _ptr(src), spitch, width, height))

    def synchronize(self):
        self._check(self._lib.galois_hip_synchronize(self._ctx))

    def event(self):
        ev = C.c_void_p()
        self._check(self._lib.galois_hip_event_create(self._ctx, C.byref(ev)))
        return ev

    def record(self, ev):
        self._check(self._lib.galois_hip_event_record(self._ctx, ev))

    def elapsed_ms(self, start, stop):
        ms = C.c_float()
        self._check(self._lib.galois_hip_event_elapsed_ms(self._ctx, start, stop, C.byref(ms)))
        return ms.value

    def event_destroy(self, ev):
        self._check(self._lib.galois_hip_event_destroy(self._ctx, ev))

    # -- stream capture ------------------------------------------------------------------
    def graph_begin_capture(self):
        self._check(self._lib.galois_hip_graph_begin_capture(self._ctx))

    def graph_end_capture(self):
        g = C.c_void_p()
        self._check(self._lib.galois_hip_graph_end_capture(self._ctx, C.byref(g)))
        return g

    def graph_launch(self, graph):
        self._check(self._lib.galois_hip_graph_launch(self._ctx, graph))

    def graph_destroy(self, graph):
        self._check(self._lib.galois_hip_graph_destroy(self._ctx, graph))

    # -- ops: same argument order as the C ABI ----------------------------------------
    def quantize_row_q4_0(self, x, y, k):
        self._check(self._lib.galois_hip_quantize_row_q4_0(self._ctx, _ptr(x), _ptr(y), k))

    def dequantize_row_q4_0(self, x, y, k):
        self._check(self._lib.galois_hip_dequantize_row_q4_0(self._ctx, _ptr(x), _ptr(y), k))

    def dequantize_mul_mat_vec_q4_0(self, vx, y, dst, ncols, nrows):
        self._check(self._lib.galois_hip_dequantize_mul_mat_vec_q4_0(self._ctx, _ptr(vx), _ptr(y), _ptr(dst),
                                                                     ncols, nrows))

    @staticmethod
    def gemv_items(items):
        """galois_hip_gemv_item array from dicts with vx, y, dst, ncols, nrows and optionally vx_up,
        norm_weight, norm_eps, residual, dst_scaled + scale_weight, sumsq_out, sumsq_in (build it once when the same
        launch is repeated)."""
        arr = (_abi.GemvItem * max(1, len(items)))()
        for a, it in zip(arr, items):
            a.vx, a.y, a.dst = _ptr(it["vx"]), _ptr(it["y"]), _ptr(it["dst"])
            a.vx_up, a.norm_weight = _ptr(it.get("vx_up")), _ptr(it.get("norm_weight"))
            a.residual = _ptr(it.get("residual"))
            a.dst_scaled, a.scale_weight = _ptr(it.get("dst_scaled")), _ptr(it.get("scale_weight"))
            a.sumsq_out, a.sumsq_in = _ptr(it.get("sumsq_out")), _ptr(it.get("sumsq_in"))
            a.ncols, a.nrows, a.norm_eps = it["ncols"], it["nrows"], it.get("norm_eps", 0.0)
        arr.n_items = len(items)
        return arr

    def dequantize_mul_mat_vec_q4_0_group(self, items):
        arr = items if isinstance(items, C.Array) else self.gemv_items(items)
        self._check(self._lib.galois_hip_dequantize_mul_mat_vec_q4_0_group(self._ctx, arr, arr.n_items))

    def mul_mat_q4_0_f32(self, W, X, Y, K, N, M):
        self._check(self._lib.galois_hip_mul_mat_q4_0_f32(self._ctx, _ptr(W), _ptr(X), _ptr(Y), K, N, M))

    def f16_panel_bytes(self, K, M):
        n = C.c_int64()
        self._check(self._lib.galois_hip_f16_panel_bytes(K, M, C.byref(n)))
        return n.value

    def f32_to_f16_panel(self, x, panel, ncols, nrows):
        self._check(self._lib.galois_hip_f32_to_f16_panel(self._ctx, _ptr(x), _ptr(panel), ncols, nrows))

    def rms_norm_mul_f16_panel(self, x, weight, panel, ncols, nrows, eps):
        self._check(self._lib.galois_hip_rms_norm_mul_f16_panel(self._ctx, _ptr(x), _ptr(weight), _ptr(panel), ncols,
                                                                nrows, eps))

    def silu_mul_f16_panel(self, gate, up, panel, ncols, nrows):
        self._check(self._lib.galois_hip_silu_mul_f16_panel(self._ctx, _ptr(gate), _ptr(up), _ptr(panel), ncols, nrows))

    def mul_mat_q4_0_f16_panel(self, items, panel, K, M):
        """items: [(W, Y, N), ...] (1 to 4 matrices against the same panel, one launch)."""
        arr = (_abi.GemmItem * len(items))()
        for a, (w, y, n) in zip(arr, items):
            a.W, a.Y, a.N = _ptr(w), _ptr(y), n
        self._check(self._lib.galois_hip_mul_mat_q4_0_f16_panel(self._ctx, arr, len(items), _ptr(panel), K, M))

    def rms_norm_f32(self, x, dst, ncols, nrows, eps):
        self._check(self._lib.galois_hip_rms_norm_f32(self._ctx, _ptr(x), _ptr(dst), ncols, nrows, eps))

    def rms_norm_mul_f32(self, x, weight, dst, ncols, nrows, eps):
        self._check(self._lib.galois_hip_rms_norm_mul_f32(self._ctx, _ptr(x), _ptr(weight), _ptr(dst), ncols, nrows,
                                                          eps))

    def rope_f32(self, x, dst, ncols, nrows, pos, freq_scale, p_delta_rows, theta_scale):
        self._check(self._lib.galois_hip_rope_f32(self._ctx, _ptr(x), _ptr(dst), ncols, nrows, _ptr(pos), freq_scale,
                                                  p_delta_rows, theta_scale))

    def soft_max_f32(self, x, dst, ncols, nrows):
        self._check(self._lib.galois_hip_soft_max_f32(self._ctx, _ptr(x), _ptr(dst), ncols, nrows))

    def soft_max_causal_f32(self, x, dst, ncols, rows_per_head, nrows, n_past):
        self._check(self._lib.galois_hip_soft_max_causal_f32(self._ctx, _ptr(x), _ptr(dst), ncols, rows_per_head,
                                                             nrows, n_past))

    def add_f32(self, x, y, dst, kx, ky):
        self._check(self._lib.galois_hip_add_f32(self._ctx, _ptr(x), _ptr(y), _ptr(dst), kx, ky))

    def mul_f32(self, x, y, dst, kx, ky):
        self._check(self._lib.galois_hip_mul_f32(self._ctx, _ptr(x), _ptr(y), _ptr(dst), kx, ky))

    def scale_f32(self, x, dst, scale, k):
        self._check(self._lib.galois_hip_scale_f32(self._ctx, _ptr(x), _ptr(dst), scale, k))

    def silu_f32(self, x, dst, k):
        self._check(self._lib.galois_hip_silu_f32(self._ctx, _ptr(x), _ptr(dst), k))

    def silu_mul_f32(self, gate, up, dst, k):
        self._check(self._lib.galois_hip_silu_mul_f32(self._ctx, _ptr(gate), _ptr(up), _ptr(dst), k))

    def cpy_f32(self, x, dst, dst_is_f16, ne, ne00, ne01, nb00, nb01, nb02, ne10, ne11, nb10, nb11, nb12):
        self._check(self._lib.galois_hip_cpy_f32(self._ctx, _ptr(x), _ptr(dst), int(dst_is_f16), ne, ne00, ne01, nb00,
                                                 nb01, nb02, ne10, ne11, nb10, nb11, nb12))

    def get_rows_q4_0(self, table, ids, dst, ncols, nr, n_table_rows):
        self._check(self._lib.galois_hip_get_rows_q4_0(self._ctx, _ptr(table), _ptr(ids), _ptr(dst), ncols, nr,
                                                       n_table_rows))

    def attn_decode_f32(self, q, k, v, k_cache, v_cache, out, n_head, head_dim, n_past, pos, freq_scale, theta_scale,
                        scale, head_major_n_ctx=0):
        self._check(self._lib.galois_hip_attn_decode_f32(self._ctx, _ptr(q), _ptr(k), _ptr(v), _ptr(k_cache),
                                                         _ptr(v_cache), _ptr(out), n_head, head_dim, n_past, _ptr(pos),
                                                         freq_scale, theta_scale, scale, head_major_n_ctx))

    def attn_decode_f32_static(self, q, k, v, k_cache, v_cache, out, n_head, head_dim, n_past, pos, freq_scale,
                               theta_scale, scale, head_major_n_ctx=0):
        self._check(self._lib.galois_hip_attn_decode_f32_static(self._ctx, _ptr(q), _ptr(k), _ptr(v), _ptr(k_cache),
                                                                _ptr(v_cache), _ptr(out), n_head, head_dim, n_past,
                                                                _ptr(pos), freq_scale, theta_scale, scale,
                                                                head_major_n_ctx))

    def qkv_attn_decode(self, items, k_cache, v_cache, out, n_head, head_dim, n_past, pos, freq_scale, theta_scale, scale,
                        kv_f16=False, head_major_n_ctx=0):
        """The three q | k | v products (gemv_items of length 3) and the decode attention in one launch."""
        arr = items if isinstance(items, C.Array) else self.gemv_items(items)
        fn = self._lib.galois_hip_qkv_attn_decode_f16kv if kv_f16 else self._lib.galois_hip_qkv_attn_decode_f32
        self._check(fn(self._ctx, arr, _ptr(k_cache), _ptr(v_cache), _ptr(out), n_head, head_dim, n_past, _ptr(pos),
                       freq_scale, theta_scale, scale, head_major_n_ctx))

    def mul_mat_q4_0_f16_panel_add(self, W, panel, residual, Y, K, N, M, workspace=None, workspace_bytes=0):
        """Y = residual + W . panel (residual may be None); with a workspace of 2 * M * N floats a matrix too narrow
        for the device is multiplied as two shares of k."""
        self._check(self._lib.galois_hip_mul_mat_q4_0_f16_panel_add(self._ctx, _ptr(W), _ptr(panel), _ptr(residual), _ptr(Y), K, N, M,
                                                                    _ptr(workspace), workspace_bytes))

    def mul_mat_q4_0_swiglu_f16_panel(self, W_gate, W_up, panel, panel_out, K, N, M):
        """panel_out = the panel of silu(W_gate . x) * (W_up . x) for x given as `panel`, one launch."""
        self._check(self._lib.galois_hip_mul_mat_q4_0_swiglu_f16_panel(self._ctx, _ptr(W_gate), _ptr(W_up), _ptr(panel), _ptr(panel_out),
                                                                       K, N, M))

    def mul_mat_q4_0_f16_panel_shares(self, W, panel, shares, shares_bytes, K, N, M):
        """W . panel as one or two partial results (M * N floats apart) in `shares`; returns how many."""
        n = C.c_int32(0)
        self._check(self._lib.galois_hip_mul_mat_q4_0_f16_panel_shares(self._ctx, _ptr(W), _ptr(panel), _ptr(shares), shares_bytes,
                                                                       K, N, M, C.byref(n)))
        return n.value

    def add_rms_norm_mul_f16_panel(self, a, b, c, sum_out, weight, panel, ncols, nrows, eps):
        """sum_out = a (+ b) (+ c); rms_norm(sum_out, eps) * weight into the panel."""
        self._check(self._lib.galois_hip_add_rms_norm_mul_f16_panel(self._ctx, _ptr(a), _ptr(b), _ptr(c), _ptr(sum_out), _ptr(weight),
                                                                    _ptr(panel), ncols, nrows, eps))

    def rope_qk_append(self, q, k, v, q_out, k_rows, v_rows, kv_f16, head_dim, n_head, n_tokens, pos, freq_scale, theta_scale):
        """rope of q (to q_out) and of k (to the cache rows k_rows) and, when v is given, v to v_rows, one launch."""
        self._check(self._lib.galois_hip_rope_qk_append(self._ctx, _ptr(q), _ptr(k), _ptr(v), _ptr(q_out), _ptr(k_rows), _ptr(v_rows),
                                                        int(kv_f16), head_dim, n_head, n_tokens, _ptr(pos), freq_scale, theta_scale))

    def attn_prefill(self, q, k_cache, v_cache, out, out_panel, n_head, head_dim, n_tokens, n_past, scale, kv_f16=False):
        """Causal attention of n_tokens rows of q over caches that already hold positions 0 .. n_past + n_tokens - 1;
        the result goes to out (f32) or out_panel (fp16 panel), the other is None."""
        fn = self._lib.galois_hip_attn_prefill_f16kv if kv_f16 else self._lib.galois_hip_attn_prefill_f32
        self._check(fn(self._ctx, _ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(out) if out is not None else None,
                       _ptr(out_panel) if out_panel is not None else None, n_head, head_dim, n_tokens, n_past, scale))

    def attn_decode_f16kv(self, q, k, v, k_cache, v_cache, out, n_head, head_dim, n_past, pos, freq_scale, theta_scale,
                          scale, head_major_n_ctx=0):
        self._check(self._lib.galois_hip_attn_decode_f16kv(self._ctx, _ptr(q), _ptr(k), _ptr(v), _ptr(k_cache),
                                                           _ptr(v_cache), _ptr(out), n_head, head_dim, n_past,
                                                           _ptr(pos), freq_scale, theta_scale, scale, head_major_n_ctx))

    def mul_mat_f16_f32(self, a, b, dst, K, N, M, ne02, ne12, a_s0, a_s1, a_s2):
        self._check(self._lib.galois_hip_mul_mat_f16_f32(self._ctx, _ptr(a), _ptr(b), _ptr(dst), K, N, M, ne02, ne12,
                                                         a_s0, a_s1, a_s2))

    def mul_mat_f32(self, a, b, dst, K, N, M, ne02, ne12, a_s0, a_s1, a_s2):
        self._check(self._lib.galois_hip_mul_mat_f32(self._ctx, _ptr(a), _ptr(b), _ptr(dst), K, N, M, ne02, ne12,
                                                     a_s0, a_s1, a_s2))
