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


def test_status_strings_without_device():
    lib = _abi.load()
    assert lib.galois_hip_status_string(0) == b"ok"
    for code in (-1, -2, -3, -4, -5, -6):
        assert lib.galois_hip_status_string(code) not in (b"", b"unknown status")
    assert lib.galois_hip_status_string(-99) == b"unknown status"


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
