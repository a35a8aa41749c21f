"""The host-side code under the address and undefined-behaviour sanitizers (CPU only, never on a GPU box's device).

libgalois_host.so parses untrusted model files and does raw pointer arithmetic over tensor views, and the oracle is
the checker every parity claim leans on: both are rebuilt with -fsanitize=address,undefined and the CPU tests that
drive them (the GGUF reader over every truncation point and malformed header, the host mirror's CPU tensors, the
oracle's own pins) are run again in a child interpreter that has the sanitizer runtime preloaded.  Any report aborts
the child (abort_on_error, -fno-sanitize-recover), which fails this test with the report in its message.
"""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _runtime(name):
    path = subprocess.check_output(["gcc", "-print-file-name=" + name], text=True).strip()
    assert os.path.isabs(path) and os.path.exists(path), "gcc has no %s" % name
    return path


def test_host_mirror_and_oracle_under_asan_and_ubsan():
    sys.path.insert(0, ROOT)
    from galois_amd import build as hip_build
    host_san = hip_build.build_host_sanitized()
    subprocess.check_call(["make", "-s", "-C", os.path.join(ROOT, "oracle"), "sanitize"])
    oracle_san = os.path.join(ROOT, "oracle", "_san", "libgalois_oracle.so")
    assert os.path.exists(oracle_san)
    env = dict(os.environ)
    preload = [_runtime("libasan.so"), _runtime("libubsan.so")] + [p for p in env.get("LD_PRELOAD", "").split(":") if p]
    env.update(LD_PRELOAD=":".join(preload), GALOIS_HOST_LIB=host_san, GALOIS_ORACLE_LIB=oracle_san,
               # leaks: the interpreter itself never frees most of what it allocates
               ASAN_OPTIONS="detect_leaks=0:abort_on_error=1:halt_on_error=1",
               UBSAN_OPTIONS="print_stacktrace=1:halt_on_error=1")
    probe = ("import os, ctypes; from galois_amd import host_api; import oracle; host_api.lib(); oracle.lib();"
             "m = open('/proc/self/maps').read();"
             "assert os.environ['GALOIS_HOST_LIB'] in m and os.environ['GALOIS_ORACLE_LIB'] in m and 'libasan' in m;"
             "print('sanitized libraries loaded')")
    r = subprocess.run([sys.executable, "-c", probe], cwd=ROOT, env=env, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0 and "sanitized libraries loaded" in r.stdout, r.stdout + r.stderr
    r = subprocess.run([sys.executable, "-m", "pytest", "-x", "-q", "-m", "not gpu", "-p", "no:cacheprovider",
                        "tests/test_gguf.py", "tests/test_oracle.py", "tests/test_xprep.py",
                        "tests/test_abi.py::test_host_mirror_builds_and_uses_only_the_c_abi"],
                       cwd=ROOT, env=env, capture_output=True, text=True, timeout=1500)
    tail = (r.stdout + r.stderr)[-4000:]
    assert r.returncode == 0, tail
    assert "AddressSanitizer" not in tail and "runtime error" not in tail, tail
