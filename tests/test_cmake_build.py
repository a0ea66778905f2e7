"""The CMake build (HIP language, gfx950 only) stands where the reference has its CUDA CMakeLists.txt
(CMakeLists.txt:1-127, one executable at :115-123).  Nothing else in the suite uses it - the tests load the library that
build.py compiles with one hipcc line - so this test configures and builds it into a scratch directory and checks that
the shared library it produces exports every symbol the headers declare.  Cross-compilation only: no GPU needed."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG_DIR = os.path.join(ROOT, "int8-flash-attention-fmha-quantization_amd")


@pytest.mark.skipif(shutil.which("cmake") is None or shutil.which("ninja") is None, reason="cmake and ninja needed")
def test_cmake_configures_builds_and_exports_the_c_abi(pkg, tmp_path):
    build = str(tmp_path / "build")
    env = dict(os.environ, CMAKE_BUILD_PARALLEL_LEVEL=os.environ.get("CMAKE_BUILD_PARALLEL_LEVEL", "8"))
    for cmd in (["cmake", "-S", PKG_DIR, "-B", build, "-G", "Ninja"], ["cmake", "--build", build]):
        r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, env=env)
        assert r.returncode == 0, " ".join(cmd) + "\n" + r.stdout[-4000:]
    lib = os.path.join(build, "libfmha_i8.so")
    assert os.path.exists(lib) and os.path.exists(os.path.join(build, "test_fmha_i8"))
    nm = subprocess.run(["nm", "-D", "--defined-only", lib], stdout=subprocess.PIPE, text=True, check=True).stdout
    exported = {line.split()[-1] for line in nm.splitlines() if line.strip()}
    missing = [s for s in pkg.EXPORTED_SYMBOLS if s not in exported]
    assert not missing, missing
    # gfx950 code objects only: the library's fat binary names no other target
    targets = subprocess.run(["strings", "-n", "8", lib], stdout=subprocess.PIPE, text=True, check=True).stdout
    assert "amdgcn-amd-amdhsa--gfx950" in targets
    assert not any(t in targets for t in ("--gfx90a", "--gfx942", "--gfx1100"))
