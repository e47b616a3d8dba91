"""Builds and calls oracle/bert_layer_loops.cpp: the BERT encoder layer forward + backward as C++ / OpenMP loop nests.

TEST AND MEASUREMENT INFRASTRUCTURE ONLY (the CPU baseline timed by bench.py; pinned against oracle/bert_layer.py in
tests/test_oracle.py). ``python -m oracle.bert_layer_loops`` builds the shared library in place.
"""
import ctypes
import os
import shutil
import subprocess

import numpy as np

from .bert_layer import PARAM_NAMES

HERE = os.path.dirname(os.path.abspath(__file__))
SRC = os.path.join(HERE, "bert_layer_loops.cpp")
LIB = os.path.join(HERE, "_build", "libbert_layer_loops.so")
# AVX2 + FMA rather than -march=native: the library is built on one machine and timed on another
FLAGS = ["-O3", "-std=c++17", "-fopenmp", "-mavx2", "-mfma", "-fno-math-errno", "-shared", "-fPIC"]

_lib = None


def build() -> str:
    cxx = shutil.which("g++")
    if cxx is None:
        raise RuntimeError("g++ not found")
    os.makedirs(os.path.dirname(LIB), exist_ok=True)
    res = subprocess.run([cxx, *FLAGS, SRC, "-o", LIB], capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("compiling %s failed:\n%s" % (SRC, res.stderr[-4000:]))
    return LIB


def load():
    """The built library (built first when it is missing or older than its source)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB) or os.path.getmtime(LIB) < os.path.getmtime(SRC):
            build()
        lib = ctypes.CDLL(LIB)
        fpp = ctypes.POINTER(ctypes.c_void_p)
        lib.bert_layer_loops.argtypes = [ctypes.c_void_p, ctypes.c_void_p, fpp, ctypes.c_void_p, ctypes.c_void_p, fpp] + \
            [ctypes.c_int] * 5 + [ctypes.c_float]
        lib.bert_layer_loops.restype = ctypes.c_int
        lib.bert_layer_loops_threads.restype = ctypes.c_int
        _lib = lib
    return _lib


def threads() -> int:
    return int(load().bert_layer_loops_threads())


def forward_backward(x, p, heads, dy=None, eps=1e-12):
    """fp32 in, fp32 out. Returns ``(y, grads)``; ``grads`` (keys ``x`` and PARAM_NAMES) is None without ``dy``."""
    lib = load()
    x = np.ascontiguousarray(x, dtype=np.float32)
    params = [np.ascontiguousarray(p[n], dtype=np.float32) for n in PARAM_NAMES]
    bsz, seq, hidden = x.shape
    ffn = params[PARAM_NAMES.index("ffn1_w")].shape[0]
    y = np.empty_like(x)
    ptrs = (ctypes.c_void_p * len(params))(*[a.ctypes.data for a in params])
    if dy is None:
        rc = lib.bert_layer_loops(x.ctypes.data, None, ptrs, y.ctypes.data, None, None, bsz, seq, hidden, heads, ffn, eps)
        grads = None
    else:
        dy = np.ascontiguousarray(dy, dtype=np.float32)
        assert dy.shape == x.shape
        dx = np.empty_like(x)
        gs = [np.empty_like(a) for a in params]
        gptrs = (ctypes.c_void_p * len(gs))(*[a.ctypes.data for a in gs])
        rc = lib.bert_layer_loops(x.ctypes.data, dy.ctypes.data, ptrs, y.ctypes.data, dx.ctypes.data, gptrs, bsz, seq, hidden,
                                  heads, ffn, eps)
        grads = dict(zip(PARAM_NAMES, gs), x=dx)
    if rc != 0:
        raise ValueError("bert_layer_loops refused the shapes %s / heads %d" % (x.shape, heads))
    return y, grads


if __name__ == "__main__":
    print(build())
