"""Build recipe of libfmha_i8.so: one hipcc line, gfx950 only, output in-tree beside this file."""
import os
import shutil
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
LIB_PATH = os.path.join(HERE, "libfmha_i8.so")
SOURCES = [os.path.join(HERE, "csrc", "fmha_i8_api.hip"), os.path.join(HERE, "csrc", "fmha_quant.hip")]
DEPENDS = SOURCES + [os.path.join(HERE, "csrc", "fmha_i8_kernel.hip"), os.path.join(HERE, "csrc", "fmha_i8_test_builds.h"),
                     os.path.join(ROOT, "include", "fmha_i8.h"), os.path.join(ROOT, "include", "fmha_param_i8.h"),
                     os.path.join(ROOT, "include", "fmha_quant.h")]
# Packed-FP32 instruction selection is switched off for all device code (a flag for hipcc's device pass; the host pass
# prints a harmless "not a recognized feature" note).
HIPCC_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def hipcc_path():
    return shutil.which("hipcc") or "/opt/rocm/bin/hipcc"


def build_library(verbose=False):
    """Compile the kernel and the C ABI into libfmha_i8.so (always recompiles)."""
    cmd = [hipcc_path()] + HIPCC_FLAGS + ["-I", os.path.join(ROOT, "include"), "-o", LIB_PATH] + SOURCES
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l)
    if proc.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + " ".join(cmd) + "\n" + out)
    if verbose and out.strip():
        print(out)
    return LIB_PATH


def is_stale():
    if not os.path.exists(LIB_PATH):
        return True
    t = os.path.getmtime(LIB_PATH)
    return any(os.path.getmtime(p) > t for p in DEPENDS)


if __name__ == "__main__":
    print(build_library(verbose=True))
