"""The build-side binding shown to maintainers (the prebuilt library as an imported CMake target that the
reference's `kernels` library links) as a project of its own, tests/cmake/CMakeLists.txt: it must configure, and
the reference's call sites (tests/cpp/test_reference_callsites.cpp) must compile and link against it.  No GPU is
needed to build; the same source runs on the GPU through tests/test_gpu_cpp_host.py."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_cmake_imported_target_builds_the_reference_call_sites(B, O, tmp_path):
    if not shutil.which("cmake"):
        pytest.skip("cmake is not installed")
    B.load()                                                     # makes sure the library is built
    gen = ["-G", "Ninja"] if shutil.which("ninja") else []
    build = str(tmp_path / "build")
    cfg = subprocess.run(["cmake", "-S", os.path.join(ROOT, "tests", "cmake"), "-B", build, "-DRLX_ROOT=" + ROOT] + gen,
                         capture_output=True, text=True, timeout=120)
    assert cfg.returncode == 0, cfg.stdout + cfg.stderr
    res = subprocess.run(["cmake", "--build", build], capture_output=True, text=True, timeout=300)
    assert res.returncode == 0, res.stdout + res.stderr
    exe = os.path.join(build, "test_reference_callsites")
    assert os.path.exists(exe)
    deps = subprocess.run(["ldd", exe], capture_output=True, text=True).stdout
    assert "librlx_adamw.so" in deps and "not found" not in deps, deps
