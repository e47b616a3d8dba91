"""Compile tests/cabi/gemm_from_cpp.cpp against the public header and the built library, and the stand-alone measurement
program tests/cabi/simd_issue_probe.hip (no library: what one SIMD does with MFMA / vector / LDS instruction mixes).

Usage: ``python tests/cabi/build.py``. The executables are written next to the sources (git-ignored)."""
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


def build_probe() -> str:
    exe = os.path.join(HERE, "simd_issue_probe")
    cmd = ["hipcc", "-O3", "--offload-arch=gfx950", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
           "-Wno-unused-command-line-argument", os.path.join(HERE, "simd_issue_probe.hip"), "-o", exe]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("compiling simd_issue_probe.hip failed:\n%s" % res.stderr[-4000:])
    return exe


if __name__ == "__main__":
    print(build())
    print(build_probe())
    sys.exit(0)
