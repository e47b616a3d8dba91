"""Compile tests/cabi/gemm_from_cpp.cpp against the public header and the built library.

Usage: ``python tests/cabi/build.py``. The executable is written next to the source (git-ignored)."""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
LIB_DIR = os.path.join(ROOT, "daceml_amd", "csrc")
EXE = os.path.join(HERE, "gemm_from_cpp")


def build() -> str:
    if not os.path.exists(os.path.join(LIB_DIR, "libdaceml_hip.so")):
        raise RuntimeError("build libdaceml_hip.so first (python -m daceml_amd.csrc.build)")
    cmd = ["hipcc", "-O2", "--offload-arch=gfx950", os.path.join(HERE, "gemm_from_cpp.cpp"), "-o", EXE,
           "-I" + os.path.join(ROOT, "include"), "-L" + LIB_DIR, "-ldaceml_hip",
           "-Wl,-rpath,$ORIGIN/" + os.path.relpath(LIB_DIR, HERE), "-Wno-unused-result"]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("compiling gemm_from_cpp.cpp failed:\n%s" % res.stderr[-4000:])
    return EXE


if __name__ == "__main__":
    print(build())
    sys.exit(0)
