"""CPU-only checks of the drop-in boundary: the header, the built library and the ctypes
declarations agree symbol for symbol.  No compute call is made (no GPU here)."""
import ctypes as C
import os
import re
import subprocess

import pytest

from galois_amd import _abi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "galois_hip.h")


def _declared():
    src = open(HEADER).read()
    src = re.sub(r"/\*.*?\*/", "", src, flags=re.S)
    return sorted(set(re.findall(r"\b(galois_hip_[a-z0-9_]+)\s*\(", src)))


def test_header_declares_something():
    names = _declared()
    assert "galois_hip_dequantize_mul_mat_vec_q4_0" in names
    assert "galois_hip_mul_mat_q4_0_f32" in names
    assert len(names) >= 20


def test_library_exports_every_declared_symbol():
    assert os.path.exists(_abi.LIB_PATH), "build first: python -m galois_amd.build"
    lib = C.CDLL(_abi.LIB_PATH)
    for name in _declared():
        assert hasattr(lib, name), name


def test_ctypes_prototypes_cover_header_exactly():
    assert sorted(_abi.PROTOTYPES) == _declared()


def _c_prototypes():
    """name -> (return class, [argument class, ...]) from the header text.  Classes: i32, i64, f32, size, ptr."""
    src = open(HEADER).read()
    src = re.sub(r"/\*.*?\*/", "", src, flags=re.S)

    def cls(t):
        t = t.strip()
        if "*" in t:
            return "ptr"
        t = re.sub(r"\bconst\b", "", t).split()
        base = t[0] if t[0] in ("int32_t", "int64_t", "float", "size_t") else None
        assert base, t
        return {"int32_t": "i32", "int64_t": "i64", "float": "f32", "size_t": "size"}[base]

    out = {}
    for ret, name, args in re.findall(r"\n((?:const\s+)?[a-z0-9_]+\s*\*?)\s*(galois_hip_[a-z0-9_]+)\s*\(([^;{]*?)\)\s*;", src):
        argl = [] if args.strip() in ("", "void") else [cls(a) for a in args.split(",")]
        out[name] = (cls(ret), argl)
    return out


def _ctypes_class(t):
    if t in (C.c_int32,):
        return "i32"
    if t in (C.c_int64,):
        return "i64"
    if t is C.c_float:
        return "f32"
    if t is C.c_size_t:
        return "size"
    return "ptr"  # c_void_p, c_char_p, POINTER(...)


def test_ctypes_argument_lists_match_the_header():
    cproto = _c_prototypes()
    assert sorted(cproto) == _declared()
    for name, (res, args) in _abi.PROTOTYPES.items():
        cres, cargs = cproto[name]
        assert [_ctypes_class(a) for a in args] == cargs, name
        assert _ctypes_class(res) == cres, name


def _rust_prototypes():
    """The Rust extern block of the integration notes: the binding a maintainer would paste into src/hip.rs."""
    text = open(os.path.join(ROOT, "INTEGRATION.md")).read()
    out = {}
    for name, args, ret in re.findall(r"pub fn (galois_hip_[a-z0-9_]+)\(([^)]*)\)\s*->\s*([^;]+);", text):
        def cls(t):
            t = t.split(":", 1)[1].strip()
            if t.startswith("*"):
                return "ptr"
            return {"i32": "i32", "i64": "i64", "f32": "f32", "usize": "size"}[t]
        argl = [cls(a) for a in args.split(",") if a.strip()]
        out[name] = ("ptr" if ret.strip().startswith("*") else {"i32": "i32"}[ret.strip()], argl)
    return out


def test_rust_binding_block_matches_the_header():
    rust, cproto = _rust_prototypes(), _c_prototypes()
    assert sorted(rust) == sorted(cproto), sorted(set(cproto) ^ set(rust))
    for name, sig in rust.items():
        assert sig == cproto[name], name
    # the struct of the grouped launch, field for field
    text = open(os.path.join(ROOT, "INTEGRATION.md")).read()
    body = re.search(r"pub struct GaloisHipGemvItem \{(.*?)\}", text, flags=re.S).group(1)
    body = re.sub(r"//[^\n]*", "", body)
    rust_fields = [f.strip().split(":")[0].replace("pub ", "").strip() for f in body.replace("\n", " ").split(",") if ":" in f]
    assert rust_fields == [f[0] for f in _abi.GemvItem._fields_]
    hsrc = re.sub(r"/\*.*?\*/", "", open(HEADER).read(), flags=re.S)
    cbody = re.search(r"typedef struct galois_hip_gemv_item \{(.*?)\}", hsrc, flags=re.S).group(1)
    c_fields = []
    for decl in cbody.split(";"):
        decl = decl.strip()
        if decl:
            c_fields += [re.sub(r"[*\s]", "", n.split()[-1]) for n in decl.split(",")]
    assert c_fields == rust_fields


def test_status_strings_without_device():
    lib = _abi.load()
    assert lib.galois_hip_status_string(0) == b"ok"
    for code in (-1, -2, -3, -4, -5, -6, -7):
        assert lib.galois_hip_status_string(code) not in (b"", b"unknown status")
    assert lib.galois_hip_status_string(-99) == b"unknown status"


def test_abi_version_is_exported_and_matches_the_header():
    lib = _abi.load()
    m = re.search(r"#define GALOIS_HIP_ABI_VERSION (\d+)", open(HEADER).read())
    assert lib.galois_hip_abi_version() == int(m.group(1)) == _abi.ABI_VERSION
    assert lib.galois_hip_set_option(None, 1, 1) == -1


def test_null_context_is_an_error_not_a_crash():
    lib = _abi.load()
    assert lib.galois_hip_synchronize(None) == -1
    assert lib.galois_hip_dequantize_mul_mat_vec_q4_0(None, None, None, None, 32, 1) == -1
    assert lib.galois_hip_mul_mat_q4_0_f32(None, None, None, None, 32, 1, 1) == -1
    assert lib.galois_hip_rms_norm_f32(None, None, None, 32, 1, 0.0) == -1
    assert lib.galois_hip_soft_max_f32(None, None, None, 32, 1) == -1
    assert lib.galois_hip_last_error(None) == b""
    assert lib.galois_hip_create(0, None) == -1


def test_header_compiles_as_c_and_cxx(tmp_path):
    for comp, ext in (("gcc", "c"), ("g++", "cc")):
        src = tmp_path / ("t." + ext)
        src.write_text('#include "galois_hip.h"\nint main(void){return GALOIS_HIP_ABI_VERSION - 1;}\n')
        subprocess.check_call([comp, "-Wall", "-Werror", "-I", os.path.join(ROOT, "include"), "-c", str(src), "-o",
                               str(tmp_path / "t.o")])


def test_product_never_touches_the_oracle():
    """The shipped package must not import, load or link anything under oracle/."""
    pkg = os.path.join(ROOT, "galois_amd")
    for dirpath, _, files in os.walk(pkg):
        if os.path.basename(dirpath) == "build":
            continue
        for f in files:
            if f.endswith((".py", ".hip", ".h", ".hpp", ".cpp", ".c")):
                text = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in text.lower(), os.path.join(dirpath, f)


def test_host_mirror_builds_and_uses_only_the_c_abi():
    """libgalois_host.so (C++ mirror of galois's op layer) links against libgalois_hip.so and nothing of HIP."""
    from galois_amd import host_api
    assert os.path.exists(host_api.LIB_PATH), "build first: python -m galois_amd.build"
    host_api.lib()
    out = subprocess.check_output(["nm", "-D", "--undefined-only", host_api.LIB_PATH], text=True)
    used = sorted(set(re.findall(r"\bgalois_hip_[a-z0-9_]+", out)))
    assert "galois_hip_dequantize_mul_mat_vec_q4_0" in used and "galois_hip_mul_mat_q4_0_f32" in used
    assert set(used) <= set(_declared())
    assert not re.search(r"\bhip[A-Z]", out), "the host mirror must not call HIP directly"
    # CPU tensors work without a GPU; GPU ops on them are 'Unimplemented', never a crash
    import numpy as np
    cpu = host_api.Device.cpu()
    t = host_api.Tensor.from_raw(np.arange(8, dtype=np.float32), [4, 2], host_api.F32, cpu)
    assert np.array_equal(t.to_cpu_tensor(), np.arange(8, dtype=np.float32).reshape(2, 4))
    with pytest.raises(host_api.GError) as e:
        host_api.galois_soft_max(t, t)
    assert e.value.kind == "Unimplemented"
