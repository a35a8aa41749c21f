"""Builds libgalois_hip.so (hand-written HIP for gfx950 + the C ABI) in-tree with hipcc.

gfx950 only: no other offload arch, no CUDA path.  Packed-FP32 instruction selection is
switched off for all device code (``-packed-fp32-ops``).
"""
import glob
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build")
LIB = os.path.join(HERE, "libgalois_hip.so")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-function",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def _compile(src, extra=()):
    obj = os.path.join(OBJ, os.path.basename(src) + ".o")
    cmd = [HIPCC, *FLAGS, *extra, "-c", src, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l and l.strip())
    if r.returncode != 0:
        raise RuntimeError("hipcc failed: %s\n%s" % (" ".join(cmd), r.stderr))
    if err:
        sys.stderr.write(err + "\n")
    return obj


def build(verbose=False, extra=()):
    os.makedirs(OBJ, exist_ok=True)
    srcs = sorted(glob.glob(os.path.join(CSRC, "*.hip")))
    with ThreadPoolExecutor(max_workers=min(8, len(srcs))) as ex:
        objs = list(ex.map(lambda s: _compile(s, extra), srcs))
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs]
    subprocess.check_call(cmd)
    if verbose:
        print("built", LIB)
    build_host(verbose)
    return LIB


HOST_LIB = os.path.join(HERE, "libgalois_host.so")


def build_host(verbose=False):
    """The C++ host mirror of galois's op layer (g++ only: it sees nothing but include/galois_hip.h)."""
    srcs = sorted(glob.glob(os.path.join(HERE, "host", "*.cpp")))
    cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-Wall", "-Wextra", "-o", HOST_LIB, *srcs,
           "-L" + HERE, "-lgalois_hip", "-Wl,-rpath,$ORIGIN"]
    subprocess.check_call(cmd)
    if verbose:
        print("built", HOST_LIB)
    return HOST_LIB


SAN_FLAGS = ["-O1", "-g", "-fno-omit-frame-pointer", "-fsanitize=address,undefined", "-fno-sanitize-recover=undefined"]


def build_host_sanitized(verbose=False):
    """The host mirror under the address and undefined-behaviour sanitizers (host code only, for CPU tests: it parses
    model files and does pointer arithmetic over tensor views).  Goes to build/san/ and is never loaded by default;
    GALOIS_HOST_LIB points an interpreter that has the sanitizer runtime preloaded at it."""
    out_dir = os.path.join(OBJ, "san")
    os.makedirs(out_dir, exist_ok=True)
    out = os.path.join(out_dir, "libgalois_host.so")
    srcs = sorted(glob.glob(os.path.join(HERE, "host", "*.cpp")))
    cmd = ["g++", "-std=c++17", "-fPIC", "-shared", "-Wall", "-Wextra", *SAN_FLAGS, "-o", out, *srcs,
           "-L" + HERE, "-lgalois_hip", "-Wl,-rpath," + HERE]
    subprocess.check_call(cmd)
    if verbose:
        print("built", out)
    return out


if __name__ == "__main__":
    build(verbose=True, extra=sys.argv[1:])
