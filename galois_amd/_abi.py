"""ctypes declarations for libgalois_hip.so, one per prototype in include/galois_hip.h."""
import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libgalois_hip.so")

c_ctx = C.c_void_p
c_ev = C.c_void_p
vp = C.c_void_p
i32 = C.c_int32
f32 = C.c_float
sz = C.c_size_t



class GemvItem(C.Structure):
    """galois_hip_gemv_item of include/galois_hip.h, field for field."""
    _fields_ = [("vx", vp), ("vx_up", vp), ("y", vp), ("norm_weight", vp), ("residual", vp), ("dst", vp),
                ("ncols", i32), ("nrows", i32), ("norm_eps", f32), ("reserved", i32), ("dst_scaled", vp),
                ("scale_weight", vp), ("sumsq_out", vp), ("sumsq_in", vp)]


class GemmItem(C.Structure):
    """galois_hip_gemm_item of include/galois_hip.h, field for field."""
    _fields_ = [("W", vp), ("Y", vp), ("N", i32), ("reserved", i32)]


# name -> (restype, argtypes); must list every function the header declares
PROTOTYPES = {
    "galois_hip_abi_version": (i32, []),
    "galois_hip_set_option": (i32, [c_ctx, i32, i32]),
    "galois_hip_create": (i32, [i32, C.POINTER(c_ctx)]),
    "galois_hip_destroy": (i32, [c_ctx]),
    "galois_hip_init_functions": (i32, [c_ctx, i32, C.POINTER(i32)]),
    "galois_hip_last_error": (C.c_char_p, [c_ctx]),
    "galois_hip_status_string": (C.c_char_p, [i32]),
    "galois_hip_device_info": (i32, [c_ctx, C.c_char_p, i32, C.c_char_p, i32, C.POINTER(i32), C.POINTER(i32),
                                     C.POINTER(i32), C.POINTER(C.c_int64)]),
    "galois_hip_alloc_zeros": (i32, [c_ctx, sz, C.POINTER(vp)]),
    "galois_hip_free": (i32, [c_ctx, vp]),
    "galois_hip_htod_sync_copy": (i32, [c_ctx, vp, vp, sz]),
    "galois_hip_dtoh_sync_copy": (i32, [c_ctx, vp, vp, sz]),
    "galois_hip_dtod_copy": (i32, [c_ctx, vp, vp, sz]),
    "galois_hip_dtod_copy_2d": (i32, [c_ctx, vp, sz, vp, sz, sz, sz]),
    "galois_hip_synchronize": (i32, [c_ctx]),
    "galois_hip_event_create": (i32, [c_ctx, C.POINTER(c_ev)]),
    "galois_hip_event_record": (i32, [c_ctx, c_ev]),
    "galois_hip_event_elapsed_ms": (i32, [c_ctx, c_ev, c_ev, C.POINTER(f32)]),
    "galois_hip_event_destroy": (i32, [c_ctx, c_ev]),
    "galois_hip_graph_begin_capture": (i32, [c_ctx]),
    "galois_hip_graph_end_capture": (i32, [c_ctx, C.POINTER(vp)]),
    "galois_hip_graph_launch": (i32, [c_ctx, vp]),
    "galois_hip_graph_destroy": (i32, [c_ctx, vp]),
    "galois_hip_quantize_row_q4_0": (i32, [c_ctx, vp, vp, C.c_int64]),
    "galois_hip_dequantize_row_q4_0": (i32, [c_ctx, vp, vp, C.c_int64]),
    "galois_hip_dequantize_mul_mat_vec_q4_0": (i32, [c_ctx, vp, vp, vp, i32, i32]),
    "galois_hip_dequantize_mul_mat_vec_q4_0_group": (i32, [c_ctx, C.POINTER(GemvItem), i32]),
    "galois_hip_mul_mat_q4_0_f32": (i32, [c_ctx, vp, vp, vp, i32, i32, i32]),
    "galois_hip_f16_panel_bytes": (i32, [i32, i32, C.POINTER(C.c_int64)]),
    "galois_hip_f32_to_f16_panel": (i32, [c_ctx, vp, vp, i32, i32]),
    "galois_hip_rms_norm_mul_f16_panel": (i32, [c_ctx, vp, vp, vp, i32, i32, f32]),
    "galois_hip_silu_mul_f16_panel": (i32, [c_ctx, vp, vp, vp, i32, i32]),
    "galois_hip_mul_mat_q4_0_f16_panel": (i32, [c_ctx, C.POINTER(GemmItem), i32, vp, i32, i32]),
    "galois_hip_rms_norm_f32": (i32, [c_ctx, vp, vp, i32, i32, f32]),
    "galois_hip_rms_norm_mul_f32": (i32, [c_ctx, vp, vp, vp, i32, i32, f32]),
    "galois_hip_rope_f32": (i32, [c_ctx, vp, vp, i32, i32, vp, f32, i32, f32]),
    "galois_hip_soft_max_f32": (i32, [c_ctx, vp, vp, i32, i32]),
    "galois_hip_soft_max_causal_f32": (i32, [c_ctx, vp, vp, i32, i32, i32, i32]),
    "galois_hip_add_f32": (i32, [c_ctx, vp, vp, vp, C.c_int64, C.c_int64]),
    "galois_hip_mul_f32": (i32, [c_ctx, vp, vp, vp, C.c_int64, C.c_int64]),
    "galois_hip_scale_f32": (i32, [c_ctx, vp, vp, f32, C.c_int64]),
    "galois_hip_silu_f32": (i32, [c_ctx, vp, vp, C.c_int64]),
    "galois_hip_silu_mul_f32": (i32, [c_ctx, vp, vp, vp, C.c_int64]),
    "galois_hip_cpy_f32": (i32, [c_ctx, vp, vp, i32] + [C.c_int64] * 11),
    "galois_hip_get_rows_q4_0": (i32, [c_ctx, vp, vp, vp, i32, i32, i32]),
    "galois_hip_attn_decode_f32": (i32, [c_ctx, vp, vp, vp, vp, vp, vp, i32, i32, i32, vp, f32, f32, f32, i32]),
    "galois_hip_attn_decode_f32_static": (i32, [c_ctx, vp, vp, vp, vp, vp, vp, i32, i32, i32, vp, f32, f32, f32, i32]),
    "galois_hip_attn_decode_f16kv": (i32, [c_ctx, vp, vp, vp, vp, vp, vp, i32, i32, i32, vp, f32, f32, f32, i32]),
    "galois_hip_qkv_attn_decode_f32": (i32, [c_ctx, C.POINTER(GemvItem), vp, vp, vp, i32, i32, i32, vp, f32, f32, f32, i32]),
    "galois_hip_mul_mat_q4_0_f16_panel_add": (i32, [c_ctx, vp, vp, vp, vp, i32, i32, i32, vp, C.c_int64]),
    "galois_hip_mul_mat_q4_0_swiglu_f16_panel": (i32, [c_ctx, vp, vp, vp, vp, i32, i32, i32]),
    "galois_hip_mul_mat_q4_0_f16_panel_shares": (i32, [c_ctx, vp, vp, vp, C.c_int64, i32, i32, i32, C.POINTER(i32)]),
    "galois_hip_add_rms_norm_mul_f16_panel": (i32, [c_ctx, vp, vp, vp, vp, vp, vp, i32, i32, f32]),
    "galois_hip_rope_qk_append": (i32, [c_ctx, vp, vp, vp, vp, vp, vp, i32, i32, i32, i32, vp, f32, f32]),
    "galois_hip_attn_prefill_f32": (i32, [c_ctx, vp, vp, vp, vp, vp, i32, i32, i32, i32, f32]),
    "galois_hip_attn_prefill_f16kv": (i32, [c_ctx, vp, vp, vp, vp, vp, i32, i32, i32, i32, f32]),
    "galois_hip_qkv_attn_decode_f16kv": (i32, [c_ctx, C.POINTER(GemvItem), vp, vp, vp, i32, i32, i32, vp, f32, f32, f32, i32]),
    "galois_hip_mul_mat_f16_f32": (i32, [c_ctx, vp, vp, vp, i32, i32, i32, i32, i32, C.c_int64, C.c_int64, C.c_int64]),
    "galois_hip_mul_mat_f32": (i32, [c_ctx, vp, vp, vp, i32, i32, i32, i32, i32, C.c_int64, C.c_int64, C.c_int64]),
}

ABI_VERSION = 2   # GALOIS_HIP_ABI_VERSION this table was written against

_lib = None


def load():
    """Loads the in-tree HIP library.  There is no fallback: a missing library is an error."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                "galois_amd: %s is missing -- build it with `python -m galois_amd.build` "
                "(hipcc, gfx950); there is no CPU fallback" % LIB_PATH)
        lib = C.CDLL(LIB_PATH)
        for name, (res, args) in PROTOTYPES.items():
            fn = getattr(lib, name)
            fn.restype, fn.argtypes = res, args
        if lib.galois_hip_abi_version() != ABI_VERSION:
            raise ImportError("galois_amd: %s has ABI version %d, these bindings are written against %d -- rebuild it"
                              % (LIB_PATH, lib.galois_hip_abi_version(), ABI_VERSION))
        _lib = lib
    return _lib
