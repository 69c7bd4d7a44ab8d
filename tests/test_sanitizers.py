"""CPU sanitizer leg: the oracle and the host-only code of the product under
AddressSanitizer + UndefinedBehaviorSanitizer (-fno-sanitize-recover: the first
finding ends the run).  Nothing here touches a GPU, and nothing sanitized is ever
sent to one."""
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SAN = ["-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=all", "-fno-omit-frame-pointer"]


def _runtime(name):
    path = subprocess.check_output(["gcc", "-print-file-name=" + name], text=True).strip()
    if not os.path.isabs(path):
        pytest.skip("%s not found next to gcc" % name)
    return path


def test_host_code_under_sanitizers(tmp_path):
    """csrc/crl_host.cpp (threaded map generators, epsilon tables, classifier, Philox) and
    host/npy.cpp (reader / writer, headers that lie about length and shape) driven by
    tests/sanitize_host.cpp."""
    exe = str(tmp_path / "sanitize_host")
    subprocess.check_call(["g++", "-std=c++17"] + SAN + ["-I", os.path.join(ROOT, "include"), "-o", exe,
                           os.path.join(ROOT, "tests", "sanitize_host.cpp"),
                           os.path.join(ROOT, "cudarl-arena_amd", "csrc", "crl_host.cpp"),
                           os.path.join(ROOT, "cudarl-arena_amd", "host", "npy.cpp"), "-lpthread"])
    out = subprocess.run([exe, str(tmp_path)], capture_output=True, text=True, timeout=300,
                         env=dict(os.environ, ASAN_OPTIONS="detect_leaks=1", UBSAN_OPTIONS="print_stacktrace=1"))
    assert out.returncode == 0, out.stdout + out.stderr
    assert "sanitize_host ok" in out.stdout


def test_oracle_pins_under_sanitizers(tmp_path):
    """Every pin of tests/test_oracle_pins.py against `make -C oracle asan`, in a child
    interpreter that has the sanitizer runtime loaded first."""
    lib = str(tmp_path / "libcrl_oracle_asan.so")
    subprocess.check_call(["make", "-s", "-B", "-C", os.path.join(ROOT, "oracle"), "asan"])
    os.replace(os.path.join(ROOT, "oracle", "libcrl_oracle_asan.so"), lib)
    preload = " ".join(p for p in (_runtime("libasan.so"), _runtime("libubsan.so"), os.environ.get("LD_PRELOAD", "")) if p)
    env = dict(os.environ, CRL_ORACLE_SO=lib, LD_PRELOAD=preload,
               # the interpreter's own allocations at exit are not the subject
               ASAN_OPTIONS="detect_leaks=0:verify_asan_link_order=0", UBSAN_OPTIONS="print_stacktrace=1")
    out = subprocess.run([sys.executable, "-m", "pytest", os.path.join(ROOT, "tests", "test_oracle_pins.py"), "-x", "-q",
                          "-p", "no:cacheprovider"], capture_output=True, text=True, timeout=900, env=env, cwd=ROOT)
    assert out.returncode == 0, out.stdout[-3000:] + out.stderr[-3000:]
    assert " passed" in out.stdout and "failed" not in out.stdout
