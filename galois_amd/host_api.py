"""ctypes face of libgalois_host.so, the C++ mirror of galois's Tensor / op interface.

Names follow the reference: ``Tensor.from_raw`` (src/lib.rs:2477), ``to_cpu_tensor``
(src/lib.rs:2279), ``galois_matmul`` / ``galois_rms_norm`` / ``galois_rope_custom`` /
``galois_soft_max`` (src/op.rs:3093-3341).  Shapes are ggml order: ne0 (innermost) first.
"""
import ctypes as C
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
# GALOIS_HOST_LIB: another build of the same library (the address / undefined-behaviour sanitizer build that
# tests/test_sanitizers.py makes with galois_amd.build.build_host_sanitized)
LIB_PATH = os.environ.get("GALOIS_HOST_LIB") or os.path.join(HERE, "libgalois_host.so")

F32, F16, Q4_0, I32 = 0, 1, 2, 18
_NP = {F32: np.float32, F16: np.float16, Q4_0: np.uint8, I32: np.int32}
KINDS = {1: "Unimplemented", 2: "ShapeError", 3: "DeviceError", 4: "Unexpected"}


class GError(RuntimeError):
    def __init__(self, kind, msg):
        super().__init__("%s: %s" % (KINDS.get(kind, kind), msg))
        self.kind = KINDS.get(kind, kind)


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError("galois_amd: %s is missing -- build with `python -m galois_amd.build`" % LIB_PATH)
        L = C.CDLL(LIB_PATH)
        vp, sz = C.c_void_p, C.c_size_t
        L.galois_host_last_error.restype = C.c_char_p
        L.galois_host_last_error_kind.restype = C.c_int
        for name, res, args in (
                ("galois_host_device_new", vp, [C.c_int]), ("galois_host_device_cpu", vp, []),
                ("galois_host_device_free", None, [vp]),
                ("galois_host_device_set_option", C.c_int, [vp, C.c_int, C.c_int]),
                ("galois_host_tensor_from_raw", vp, [vp, vp, sz, sz, C.POINTER(sz), C.c_int]),
                ("galois_host_tensor_zeros", vp, [vp, sz, C.POINTER(sz), C.c_int]),
                ("galois_host_tensor_view", vp, [vp, sz, sz, C.POINTER(sz)]),
                ("galois_host_tensor_to_cpu", C.c_int, [vp, vp, sz]), ("galois_host_tensor_nbytes", sz, [vp]),
                ("galois_host_tensor_free", None, [vp]), ("galois_host_matmul", C.c_int, [vp, vp, vp]),
                ("galois_host_rms_norm", C.c_int, [vp, vp, C.c_float]),
                ("galois_host_rope_custom", C.c_int, [sz, C.c_int, C.c_int, C.c_float, C.c_float, C.c_float, C.c_int,
                                                      vp, vp, vp]),
                ("galois_host_soft_max", C.c_int, [vp, vp]),
                ("galois_host_tensor_view_strided", vp, [vp, sz, sz, C.POINTER(sz), C.POINTER(sz)]),
                ("galois_host_tensor_write", C.c_int, [vp, vp, sz]), ("galois_host_tensor_data", vp, [vp]),
                ("galois_host_add", C.c_int, [vp, vp, vp]), ("galois_host_mul", C.c_int, [vp, vp, vp]),
                ("galois_host_unary_silu", C.c_int, [vp, vp]), ("galois_host_scale", C.c_int, [vp, vp, vp]),
                ("galois_host_cpy", C.c_int, [vp, vp]), ("galois_host_cont", C.c_int, [vp, vp]),
                ("galois_host_get_rows", C.c_int, [vp, vp, vp]),
                ("galois_host_llama_new", vp, [vp, sz, sz, sz, sz, sz, sz, C.c_float, C.c_float]),
                ("galois_host_llama_new_kv", vp, [vp, sz, sz, sz, sz, sz, sz, C.c_float, C.c_float, C.c_int]),
                ("galois_host_llama_free", None, [vp]), ("galois_host_llama_tensor", vp, [vp, C.c_char_p, C.c_int]),
                ("galois_host_llama_logits", vp, [vp]), ("galois_host_llama_ops_per_step", sz, [vp]),
                ("galois_host_llama_decode", C.c_int, [vp, C.c_int32, C.c_int32, C.c_int]),
                ("galois_host_llama_prefill", C.c_int, [vp, C.POINTER(C.c_int32), sz, C.c_int32]),
                ("galois_host_llama_ops_per_prefill", sz, [vp]),
                ("galois_host_llama_time_prefill", C.c_int, [vp, vp, C.POINTER(C.c_int32), sz, C.c_int32, C.c_int,
                                                             C.POINTER(C.c_float)]),
                ("galois_host_llama_capture", C.c_int, [vp, C.c_int32, C.c_int32, C.c_int]),
                ("galois_host_llama_replay", C.c_int, [vp]),
                ("galois_host_llama_time_replays", C.c_int, [vp, vp, C.c_int, C.POINTER(C.c_float)]),
                ("galois_host_llama_time_steps", C.c_int, [vp, vp, C.c_int32, C.c_int32, C.c_int, C.c_int,
                                                           C.POINTER(C.c_float)]),
                ("galois_host_gguf_open", vp, [C.c_char_p]), ("galois_host_gguf_close", None, [vp]),
                ("galois_host_gguf_version", C.c_uint32, [vp]), ("galois_host_gguf_alignment", sz, [vp]),
                ("galois_host_gguf_data_start", sz, [vp]), ("galois_host_gguf_n_tensors", sz, [vp]),
                ("galois_host_gguf_n_kv", sz, [vp]),
                ("galois_host_gguf_tensor_info", C.c_char_p, [vp, sz, C.POINTER(sz), C.POINTER(sz),
                                                              C.POINTER(C.c_uint32), C.POINTER(C.c_uint64),
                                                              C.POINTER(sz), C.POINTER(C.c_int)]),
                ("galois_host_gguf_get_uint", C.c_int, [vp, C.c_char_p, C.POINTER(C.c_uint64)]),
                ("galois_host_gguf_get_float", C.c_int, [vp, C.c_char_p, C.POINTER(C.c_double)]),
                ("galois_host_gguf_get_string", C.c_long, [vp, C.c_char_p, C.c_char_p, sz]),
                ("galois_host_gguf_string_array", C.c_long, [vp, C.c_char_p, sz, C.c_char_p, sz]),
                ("galois_host_gguf_load_tensor", vp, [vp, C.c_char_p, vp]),
                ("galois_host_gguf_llama_hparams", C.c_int, [vp, sz, C.POINTER(sz), C.POINTER(C.c_float)]),
                ("galois_host_llama_from_gguf", vp, [vp, vp, sz])):
            fn = getattr(L, name)
            fn.restype, fn.argtypes = res, args
        _lib = L
    return _lib


def _raise(kind=None):
    """Raises the library's last error; kind None = the kind the library recorded with it."""
    if kind is None:
        kind = lib().galois_host_last_error_kind() or 4
    raise GError(kind, lib().galois_host_last_error().decode())


def _shape(shape):
    return len(shape), (C.c_size_t * len(shape))(*shape)


class Device:
    """``Device::Cpu`` or ``Device::Gpu(CudaDevice::new(ordinal))``."""

    def __init__(self, h):
        self.h = h

    @staticmethod
    def cpu():
        return Device(lib().galois_host_device_cpu())

    @staticmethod
    def gpu(ordinal=0):
        h = lib().galois_host_device_new(ordinal)
        if not h:
            _raise(3)
        return Device(h)

    def set_option(self, option, value):
        """``galois_hip_set_option`` on the device's context (option numbers: include/galois_hip.h)."""
        _call(lib().galois_host_device_set_option(self.h, option, value))


class Tensor:
    def __init__(self, h, shape, dtype):
        self.h, self.shape, self.dtype = h, tuple(shape), dtype

    @staticmethod
    def from_raw(data, shape, dtype, device):
        """``Tensor::from_raw(bytes, n_dims, Shape::from_array(shape), dtype, &device)``."""
        data = np.ascontiguousarray(data)
        n, s = _shape(shape)
        h = lib().galois_host_tensor_from_raw(device.h, data.ctypes.data_as(C.c_void_p), data.nbytes, n, s, dtype)
        if not h:
            _raise(2)
        return Tensor(h, shape, dtype)

    @staticmethod
    def zeros(shape, dtype, device):
        n, s = _shape(shape)
        h = lib().galois_host_tensor_zeros(device.h, n, s, dtype)
        if not h:
            _raise(2)
        return Tensor(h, shape, dtype)

    def view(self, elem_offset, shape):
        n, s = _shape(shape)
        h = lib().galois_host_tensor_view(self.h, elem_offset, n, s)
        if not h:
            _raise(2)
        return Tensor(h, shape, self.dtype)

    def view_strided(self, elem_offset, shape, stride):
        """A view with explicit strides in elements (what permute / transpose give in the reference)."""
        n, sh = _shape(shape)
        _, st = _shape(stride)
        h = lib().galois_host_tensor_view_strided(self.h, elem_offset, n, sh, st)
        if not h:
            _raise(2)
        return Tensor(h, shape, self.dtype)

    def write(self, data):
        data = np.ascontiguousarray(data)
        _call(lib().galois_host_tensor_write(self.h, data.ctypes.data_as(C.c_void_p), data.nbytes))

    def data_ptr(self):
        return lib().galois_host_tensor_data(self.h)

    def to_cpu_tensor(self):
        """Host copy as a numpy array shaped [ne3..ne0] (row-major), uint8 block bytes for Q4_0."""
        nb = lib().galois_host_tensor_nbytes(self.h)
        out = np.empty(nb, np.uint8)
        st = lib().galois_host_tensor_to_cpu(self.h, out.ctypes.data_as(C.c_void_p), nb)
        if st:
            _raise(st)
        if self.dtype == Q4_0:
            return out
        return out.view(_NP[self.dtype]).reshape(tuple(reversed(self.shape)))


def _call(st):
    if st:
        _raise(st)


def galois_matmul(a, b, dst):
    _call(lib().galois_host_matmul(a.h, b.h, dst.h))


def galois_rms_norm(src, dst, eps):
    _call(lib().galois_host_rms_norm(src.h, dst.h, eps))


def galois_rope_custom(op, src0, src1, dst):
    _call(lib().galois_host_rope_custom(op["n_dims"], op.get("mode", 0), op.get("n_ctx", 0),
                                        op.get("freq_base", 10000.0), op.get("freq_scale", 1.0),
                                        op.get("xpos_base", 0.0), int(op.get("xpos_down", False)), src0.h, src1.h,
                                        dst.h))


def galois_soft_max(src, dst):
    _call(lib().galois_host_soft_max(src.h, dst.h))


def galois_add(a, b, dst):
    _call(lib().galois_host_add(a.h, b.h, dst.h))


def galois_mul(a, b, dst):
    _call(lib().galois_host_mul(a.h, b.h, dst.h))


def galois_unary_silu(src, dst):
    """``galois_unary(src, dst, UnaryOp::Silu)``."""
    _call(lib().galois_host_unary_silu(src.h, dst.h))


def galois_scale(src0, src1, dst):
    _call(lib().galois_host_scale(src0.h, src1.h, dst.h))


def galois_cpy(src, dst):
    _call(lib().galois_host_cpy(src.h, dst.h))


def galois_cont(src, dst):
    _call(lib().galois_host_cont(src.h, dst.h))


def galois_get_rows(src0, src1, dst):
    _call(lib().galois_host_get_rows(src0.h, src1.h, dst.h))


class LlamaDecoder:
    """One-token decode step of a LLaMA-architecture model issued as galois ops (galois_amd/host/llama.hpp)."""

    def __init__(self, device, n_vocab=32000, n_embd=4096, n_head=32, n_layer=32, n_ff=11008, n_ctx=2048,
                 rms_eps=1e-6, freq_base=10000.0, kv_f16=False, kv_head_major=False, _handle=None):
        self.device = device
        self.hp = dict(n_vocab=n_vocab, n_embd=n_embd, n_head=n_head, n_layer=n_layer, n_ff=n_ff, n_ctx=n_ctx,
                       rms_eps=rms_eps, freq_base=freq_base)
        self.kv_f16, self.kv_head_major = bool(kv_f16), bool(kv_head_major)
        self.h = _handle or lib().galois_host_llama_new_kv(device.h, n_vocab, n_embd, n_head, n_layer, n_ff, n_ctx,
                                                           rms_eps, freq_base, int(self.kv_f16) | 2 * int(self.kv_head_major))
        if not self.h:
            _raise(3)

    @staticmethod
    def from_gguf(gguf, device, n_ctx_max=2048):
        """A decoder with the hyper-parameters and the weights of a GGUF file (``GgufFile``)."""
        hp = gguf.llama_hparams(n_ctx_max)
        h = lib().galois_host_llama_from_gguf(gguf.h, device.h, n_ctx_max)
        if not h:
            _raise()
        hp.pop("freq_scale")
        return LlamaDecoder(device, _handle=h, **hp)

    def close(self):
        if self.h:
            lib().galois_host_llama_free(self.h)
            self.h = None

    def tensor(self, name, layer=-1):
        """Borrowed handle to a weight or cache tensor (owned by the decoder)."""
        h = lib().galois_host_llama_tensor(self.h, name.encode(), layer)
        if not h:
            _raise(4)
        hp = self.hp
        e, f, v, c = hp["n_embd"], hp["n_ff"], hp["n_vocab"], hp["n_ctx"]
        shapes = {"tok_embd": ((e, v), Q4_0), "output": ((e, v), Q4_0), "out_norm": ((e,), F32),
                  "attn_norm": ((e,), F32), "ffn_norm": ((e,), F32), "wq": ((e, e), Q4_0), "wk": ((e, e), Q4_0),
                  "wv": ((e, e), Q4_0), "wo": ((e, e), Q4_0), "w_gate": ((e, f), Q4_0), "w_up": ((e, f), Q4_0),
                  "w_down": ((f, e), Q4_0)}
        cache = (e // hp["n_head"], c, hp["n_head"]) if self.kv_head_major else (e, c)   # numpy sees [H, C, D] or [C, E]
        shapes["k_cache"] = shapes["v_cache"] = (cache, F16 if self.kv_f16 else F32)
        shape, dtype = shapes[name]
        t = Tensor(h, shape, dtype)
        t.borrowed = True
        return t

    def decode(self, token, n_past, fused=False):
        _call(lib().galois_host_llama_decode(self.h, token, n_past, int(fused)))

    def prefill(self, tokens, n_past=0):
        """All of `tokens` at positions n_past .. in one pass; afterwards the caches hold them and logits() the last one's."""
        t = np.ascontiguousarray(tokens, np.int32)
        _call(lib().galois_host_llama_prefill(self.h, t.ctypes.data_as(C.POINTER(C.c_int32)), t.size, n_past))

    def ops_per_prefill(self):
        return lib().galois_host_llama_ops_per_prefill(self.h)

    def time_prefill(self, tokens, n_past, reps):
        t = np.ascontiguousarray(tokens, np.int32)
        ms = C.c_float()
        _call(lib().galois_host_llama_time_prefill(self.h, self.device.h, t.ctypes.data_as(C.POINTER(C.c_int32)), t.size, n_past,
                                                   reps, C.byref(ms)))
        return ms.value

    def capture(self, token, n_past, fused=False):
        _call(lib().galois_host_llama_capture(self.h, token, n_past, int(fused)))

    def replay(self):
        _call(lib().galois_host_llama_replay(self.h))

    def logits(self):
        t = Tensor(lib().galois_host_llama_logits(self.h), (self.hp["n_vocab"], 1), F32)
        t.borrowed = True
        return t.to_cpu_tensor().reshape(-1)

    def ops_per_step(self):
        return lib().galois_host_llama_ops_per_step(self.h)

    def time_replays(self, n):
        ms = C.c_float()
        _call(lib().galois_host_llama_time_replays(self.h, self.device.h, n, C.byref(ms)))
        return ms.value

    def time_steps(self, token, n_past, fused, n):
        ms = C.c_float()
        _call(lib().galois_host_llama_time_steps(self.h, self.device.h, token, n_past, int(fused), n, C.byref(ms)))
        return ms.value


class GgufFile:
    """A memory-mapped GGUF model file (galois_amd/host/gguf.hpp): metadata, tensor table, tensors as ``Tensor``."""

    def __init__(self, path):
        self.h = lib().galois_host_gguf_open(os.fsencode(path))
        if not self.h:
            _raise()

    def close(self):
        if self.h:
            lib().galois_host_gguf_close(self.h)
            self.h = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    @property
    def version(self):
        return lib().galois_host_gguf_version(self.h)

    @property
    def alignment(self):
        return lib().galois_host_gguf_alignment(self.h)

    @property
    def data_start(self):
        return lib().galois_host_gguf_data_start(self.h)

    @property
    def n_kv(self):
        return lib().galois_host_gguf_n_kv(self.h)

    def tensors(self):
        """List of dicts: name, shape (ne0 first), ggml_type, offset, nbytes, supported."""
        out = []
        for i in range(lib().galois_host_gguf_n_tensors(self.h)):
            nd, shape = C.c_size_t(), (C.c_size_t * 4)()
            ty, off, nb, sup = C.c_uint32(), C.c_uint64(), C.c_size_t(), C.c_int()
            name = lib().galois_host_gguf_tensor_info(self.h, i, C.byref(nd), shape, C.byref(ty), C.byref(off),
                                                      C.byref(nb), C.byref(sup))
            out.append({"name": name.decode(), "shape": tuple(shape[:nd.value]), "ggml_type": ty.value,
                        "offset": off.value, "nbytes": nb.value, "supported": bool(sup.value)})
        return out

    def get_uint(self, key):
        v = C.c_uint64()
        return v.value if lib().galois_host_gguf_get_uint(self.h, key.encode(), C.byref(v)) else None

    def get_float(self, key):
        v = C.c_double()
        return v.value if lib().galois_host_gguf_get_float(self.h, key.encode(), C.byref(v)) else None

    def get_string(self, key):
        n = lib().galois_host_gguf_get_string(self.h, key.encode(), None, 0)
        if n < 0:
            return None
        buf = C.create_string_buffer(n + 1)
        lib().galois_host_gguf_get_string(self.h, key.encode(), buf, n + 1)
        return buf.raw[:n].decode("utf-8", "replace")

    def get_string_array(self, key):
        n = lib().galois_host_gguf_string_array(self.h, key.encode(), 0, None, 0)
        if n < 0:
            return None
        out = []
        buf = C.create_string_buffer(1 << 16)
        for i in range(n):
            m = lib().galois_host_gguf_string_array(self.h, key.encode(), i, buf, len(buf))
            out.append(buf.raw[:min(m, len(buf) - 1)].decode("utf-8", "replace"))
        return out

    def load_tensor(self, name, device):
        """``Tensor::from_raw`` on the tensor's bytes (F32, F16 and Q4_0 tensors)."""
        info = next((t for t in self.tensors() if t["name"] == name), None)
        h = lib().galois_host_gguf_load_tensor(self.h, name.encode(), device.h)
        if not h:
            _raise()
        return Tensor(h, info["shape"], info["ggml_type"])

    def llama_hparams(self, n_ctx_max=2048):
        hp, fp = (C.c_size_t * 6)(), (C.c_float * 3)()
        _call(lib().galois_host_gguf_llama_hparams(self.h, n_ctx_max, hp, fp))
        return dict(n_vocab=hp[0], n_embd=hp[1], n_head=hp[2], n_layer=hp[3], n_ff=hp[4], n_ctx=hp[5],
                    rms_eps=fp[0], freq_base=fp[1], freq_scale=fp[2])
