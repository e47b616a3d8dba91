"""Build libdaceml_hip.so (gfx950 code objects + the C ABI) in-tree with hipcc.

Usage: ``python -m daceml_amd.csrc.build [--incremental]``. The shared library is written next to
the sources so that it travels with the source tree; nothing is installed.
"""
import concurrent.futures
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_NAME = "libdaceml_hip.so"
LIB_PATH = os.path.join(HERE, LIB_NAME)
OBJ_DIR = os.path.join(HERE, "build")

SOURCES = [
    "common.cpp",
    "rowwise.hip",
    "elementwise.hip",
    "reduce.hip",
    "transpose.hip",
    "pad.hip",
    "pool.hip",
    "gemm_f16.hip",
    "gemm_f16_pipe.hip",
    "gemm_f16_pipe_ilv.hip",
    "gemm_f32.hip",
    "conv.hip",
    "conv_fused.hip", "conv_backward.hip", "conv_implicit.hip",
    "attention.hip",
    "batchnorm.hip",
]

# -packed-fp32-ops: keep the compiler from forming packed-fp32 VALU instructions.
COMMON_FLAGS = [
    "-O3", "-std=c++17", "-fPIC", "--offload-arch=gfx950", "-Xclang", "-target-feature", "-Xclang",
    "-packed-fp32-ops", "-Wno-unused-command-line-argument", "-Wno-unknown-attributes",
    # the LDS readers of lds_ops.h are [[nodiscard]]: dropping the value of one is an error, not a warning
    "-Werror=unused-result",
]


def hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; a ROCm toolchain is required to build " + LIB_NAME)
    return exe


def _compile(src: str) -> str:
    obj = os.path.join(OBJ_DIR, os.path.splitext(src)[0] + ".o")
    cmd = [hipcc(), *COMMON_FLAGS, "-x", "hip", "-c", os.path.join(HERE, src), "-o", obj]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("compiling %s failed:\n%s\n%s" % (src, " ".join(cmd), res.stderr[-8000:]))
    warnings = [l for l in res.stderr.splitlines() if "warning" in l and "packed-fp32-ops" not in l]
    if warnings:
        sys.stderr.write("\n".join(warnings[:20]) + "\n")
    return obj


def _stale(src: str) -> bool:
    """Is the object file of `src` older than the source or any header?"""
    obj = os.path.join(OBJ_DIR, os.path.splitext(src)[0] + ".o")
    if not os.path.exists(obj):
        return True
    deps = [os.path.join(HERE, src)] + [os.path.join(HERE, f) for f in os.listdir(HERE) if f.endswith(".h")]
    deps.append(os.path.join(HERE, "..", "..", "include", "daceml_hip.h"))
    return os.path.getmtime(obj) < max(os.path.getmtime(d) for d in deps)


def build(force: bool = True, jobs: int = 8) -> str:
    """Compile every source (with force=False: only those whose object file is out of date) and link the shared
    library from all object files. Returns the library path."""
    os.makedirs(OBJ_DIR, exist_ok=True)
    srcs = [s for s in SOURCES if os.path.exists(os.path.join(HERE, s))]
    todo = srcs if force else [s for s in srcs if _stale(s)]
    if not todo and os.path.exists(LIB_PATH):
        return LIB_PATH
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as pool:
        list(pool.map(_compile, todo))
    objs = [os.path.join(OBJ_DIR, os.path.splitext(s)[0] + ".o") for s in srcs]
    cmd = [hipcc(), "-shared", "-fPIC", "--offload-arch=gfx950", "-o", LIB_PATH, *objs]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("linking %s failed:\n%s" % (LIB_NAME, res.stderr[-8000:]))
    return LIB_PATH


if __name__ == "__main__":
    path = build(force="--incremental" not in sys.argv)
    print(path)
