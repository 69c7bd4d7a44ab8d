"""The CMake front end offers the reference's target names (CMakeLists.txt:76-127
upstream): configure and build it in a scratch directory and check what comes out.
No GPU needed: hipcc cross-compiles gfx950."""
import ctypes as C
import glob
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.mark.skipif(shutil.which("cmake") is None or shutil.which("ninja") is None, reason="cmake + ninja not installed")
def test_cmake_configures_and_builds_the_reference_targets(tmp_path):
    build = str(tmp_path / "build")
    gen = subprocess.run(["cmake", "-S", ROOT, "-B", build, "-G", "Ninja"], capture_output=True, text=True, timeout=300)
    assert gen.returncode == 0, gen.stdout + gen.stderr
    # building them by name fails for a name the file does not offer
    targets = ["crl_engine", "cudarl_core", "cudarl_core_python", "cudarl_app", "cudarl_train", "hip_test"]
    made = subprocess.run(["cmake", "--build", build, "-j", "8", "--target"] + targets, capture_output=True, text=True,
                          timeout=900)
    assert made.returncode == 0, made.stdout[-3000:] + made.stderr[-3000:]
    text = open(os.path.join(build, "build.ninja")).read()
    assert "build run:" in text and "build run_hip_test:" in text  # the reference's convenience targets
    for name in ("libcrl.so", "libcudarl_host.so", "cudarl_app", "cudarl_train", "hip_test"):
        assert os.path.exists(os.path.join(build, name)), name
    assert glob.glob(os.path.join(build, "cudarl_core*.so")), "pybind module cudarl_core"
    lib = C.CDLL(os.path.join(build, "libcrl.so"))
    lib.crl_version.restype = C.c_char_p
    assert lib.crl_version() == b"0.1.0"
    # the demo links against the libraries beside it and fails cleanly without a device
    if lib.crl_device_count() < 1:
        out = subprocess.run([os.path.join(build, "hip_test")], capture_output=True, text=True, timeout=60)
        assert out.returncode == 1 and "no HIP device" in out.stdout
