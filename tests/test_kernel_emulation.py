"""The hand-scheduled kernels run on the CPU, lane by lane.

tests/kernel_emulation/ compiles a kernel's own source for the host: every lane is a fibre, lanes meet at matrix
instructions, LDS transpose reads, permutes and barriers, and global -> LDS transfers land either when they issue or
only when the issuing lane waits for them (emu.h says what each extreme exposes). A result that is right under both,
for several wavefront orders, means the tile ring, the waits and the barriers of the K loop are in the right places,
fragments are read from the right stage, and the tail of the loop is handled - for every tile configuration, operand
layout and K length tried. Needs the ROCm clang as a host compiler (the kernels use its vector extensions), no GPU.
It checks the logic of the source, not the machine code: that is what the GPU tests and tests/isa_hazards.py are for."""
import ctypes
import os
import shutil
import subprocess

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EMU = os.path.join(ROOT, "tests", "kernel_emulation")
CSRC = os.path.join(ROOT, "daceml_amd", "csrc")


def _clang():
    for c in ("/opt/rocm/lib/llvm/bin/clang++", shutil.which("amdclang++"), shutil.which("clang++")):
        if c and os.path.exists(c):
            return c
    pytest.skip("no clang++ to compile the kernels for the host")


def _stage_sources(tmp, files):
    """Copies of the kernel sources with lds_ops.h swapped for its host stand-in, laid out like the repository (the
    headers include ../../include/daceml_hip.h)."""
    dst = os.path.join(tmp, "daceml_amd", "csrc")
    os.makedirs(dst, exist_ok=True)
    os.makedirs(os.path.join(tmp, "include"), exist_ok=True)
    shutil.copy(os.path.join(ROOT, "include", "daceml_hip.h"), os.path.join(tmp, "include"))
    for f in files:
        text = open(os.path.join(CSRC, f)).read().replace('#include "lds_ops.h"', '#include "lds_ops_emu.h"')
        # an LDS pointer cast to its address space is the byte offset inside LDS on the GPU; here LDS is host memory
        text = text.replace("(uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)lds", "lds_addr(lds)")
        # the one LDS read that is written as inline assembly outside lds_ops.h
        text = text.replace('asm volatile("ds_read_b128 %0, %1" : "=v"(v) : "v"(addr));', "memcpy(&v, emu::g_lds + addr, 16);")
        open(os.path.join(dst, f if not f.endswith(".hip") else f[:-4] + "_emu.h"), "w").write(text)
    shutil.copy(os.path.join(EMU, "lds_ops_emu.h"), dst)
    return dst


def _build(tmp, name, harness, files, mutate=None, defines=()):
    """`mutate`: {file: function(text) -> text} applied to the staged copies (to show that a defect is detected)."""
    src_dir = _stage_sources(tmp, files)
    for f, fn in (mutate or {}).items():
        path = os.path.join(src_dir, f)
        text = open(path).read()
        changed = fn(text)
        assert changed != text, "the mutation of %s did not apply" % f
        open(path, "w").write(changed)
    out = os.path.join(tmp, name + ".so")
    cmd = [_clang(), "-std=c++17", "-O1", "-fPIC", "-shared", "-x", "c++", "-Wno-everything", *["-D" + d for d in defines], "-I", os.path.join(EMU, "shim"),
           "-I", EMU, "-I", src_dir, os.path.join(EMU, harness), os.path.join(EMU, "emu.cpp"), "-o", out]
    res = subprocess.run(cmd, capture_output=True, text=True)
    assert res.returncode == 0, res.stderr[-6000:]
    return ctypes.CDLL(out)


@pytest.fixture(scope="module")
def gemm_lib(tmp_path_factory):
    lib = _build(str(tmp_path_factory.mktemp("emu_gemm")), "emu_gemm", "gemm_harness.cpp",
                 ["common.h", "gemm_f16_common.h", "gemm_f16_pipe.h"])
    lib.emu_gemm.restype = ctypes.c_int
    return lib


def _operand(r, rows, k, kind):
    """(memory image, logical [rows, k] matrix in fp64)."""
    x = (r.standard_normal((rows, k)) * 0.5).astype(np.float16)
    return (np.ascontiguousarray(x.T) if kind else x), x.astype(np.float64)


def _run_gemm(lib, cfg, variant, akind, bkind, m, n, k, pairs, seed, late):
    r = np.random.default_rng(1000 * cfg + 10 * variant + akind * 2 + bkind + k)
    a = [_operand(r, m, k, akind) for _ in range(pairs)]
    b = [_operand(r, n, k, bkind) for _ in range(pairs)]
    c = np.full((m, n), np.nan, dtype=np.float32)
    asum = np.full(m, np.nan, dtype=np.float32)
    pa = (ctypes.c_void_p * pairs)(*[x[0].ctypes.data for x in a])
    pb = (ctypes.c_void_p * pairs)(*[x[0].ctypes.data for x in b])
    status = lib.emu_gemm(cfg, variant, akind, bkind, m, n, k, pairs, pa, pb, c.ctypes.data_as(ctypes.c_void_p),
                          asum.ctypes.data_as(ctypes.c_void_p), seed, late)
    assert status == 0, "status %d (1 = the lanes deadlocked)" % status
    want = sum(x[1] @ y[1].T for x, y in zip(a, b))
    what = "cfg %d variant %d layouts %d%d %dx%dx%d seed %d %s" % (cfg, variant, akind, bkind, m, n, k, seed,
                                                                  "late" if late else "early")
    np.testing.assert_allclose(c, want, rtol=1e-5, atol=1e-4, err_msg=what)
    if variant == 2:
        np.testing.assert_allclose(asum, a[0][1].sum(1), rtol=1e-5, atol=1e-4, err_msg=what + " (row sums)")


LAYOUTS = [(0, 0), (0, 1), (1, 0), (1, 1)]


@pytest.mark.parametrize("cfg", [0, 1, 2, 3])
def test_the_emulation_reproduces_the_kernels_that_run_on_hardware(gemm_lib, cfg):
    """The tile configurations the library uses (validated on the GPU): if the model of the matrix instruction, the
    transpose read or the transfers were wrong, these would fail first."""
    for akind, bkind in LAYOUTS:
        for k, late in ((64, 0), (320, 1)):
            _run_gemm(gemm_lib, cfg, 0, akind, bkind, 256, 256, k, 1, seed=1, late=late)
    _run_gemm(gemm_lib, cfg, 0, 0, 1, 200, 136, 192, 1, seed=2, late=1)      # rows and columns short of a tile


@pytest.mark.parametrize("cfg", [4, 5, 6, 7, 8, 9])
@pytest.mark.parametrize("late", [0, 1])
def test_interleaved_k_loop(gemm_lib, cfg, late):
    """Configurations 4 - 7 and 9 (and 8: the plain loop on the 128 x 64 tile, whose row-contiguous operand has its own
    LDS layout, new as well): every operand layout, K from one step to more than twice the ring's depth (the loop has
    a filling part, a draining part and a last step), two wavefront orders, ragged edges."""
    for akind, bkind in LAYOUTS:
        for k in (64, 128, 192, 256, 576) if akind == bkind else (64, 192, 320):
            _run_gemm(gemm_lib, cfg, 0, akind, bkind, 256, 256, k, 1, seed=3, late=late)
    _run_gemm(gemm_lib, cfg, 0, 0, 0, 256, 256, 384, 1, seed=4, late=late)
    _run_gemm(gemm_lib, cfg, 0, 1, 0, 200, 136, 320, 1, seed=6, late=late)
    _run_gemm(gemm_lib, cfg, 0, 0, 1, 520, 264, 128, 1, seed=7, late=late)    # several tiles, the last ones ragged


def test_every_configuration_adds_in_the_same_order(gemm_lib):
    """Each accumulator receives the same matrix instructions in the same order whatever the tile shape, ring depth
    or loop form: the fp32 results of all ten configurations are identical (which the GPU tests of the interleaved
    configurations assert against the default configuration)."""
    def run(cfg, akind, bkind):
        r = np.random.default_rng(7)
        a, b = _operand(r, 256, 576, akind), _operand(r, 256, 576, bkind)
        c = np.full((256, 256), np.nan, dtype=np.float32)
        pa, pb = (ctypes.c_void_p * 1)(a[0].ctypes.data), (ctypes.c_void_p * 1)(b[0].ctypes.data)
        assert gemm_lib.emu_gemm(cfg, 0, akind, bkind, 256, 256, 576, 1, pa, pb, c.ctypes.data_as(ctypes.c_void_p), None, 1,
                                 1) == 0
        return c
    for akind, bkind in ((0, 0), (1, 0)):
        base = run(0, akind, bkind)
        for cfg in range(1, 10):
            assert np.array_equal(run(cfg, akind, bkind), base), (cfg, akind, bkind)


@pytest.mark.parametrize("cfg", [0, 3, 5, 7])
def test_operand_pairs_and_row_sums(gemm_lib, cfg):
    """The K-concatenated and row-sum forms, plain loop (0, 3) and interleaved loop (5, 7)."""
    for late in (0, 1):
        for akind, bkind in LAYOUTS:
            _run_gemm(gemm_lib, cfg, 1, akind, bkind, 128, 256, 128, 3, seed=8, late=late)
        _run_gemm(gemm_lib, cfg, 1, 0, 0, 128, 128, 64, 4, seed=9, late=late)     # one step per pair
        _run_gemm(gemm_lib, cfg, 1, 1, 1, 200, 136, 192, 2, seed=10, late=late)
        for bkind in (0, 1):
            _run_gemm(gemm_lib, cfg, 2, 1, bkind, 256, 256, 320, 1, seed=11, late=late)
        _run_gemm(gemm_lib, cfg, 2, 1, 1, 200, 136, 64, 1, seed=12, late=late)


def _fails(fn):
    try:
        fn()
    except AssertionError:
        return True
    return False


def test_a_wait_that_lets_one_tile_too_many_stay_in_flight_is_detected(tmp_path):
    """The check has teeth: with the interleaved loop's wait loosened by one tile, transfers that land late are read
    before they arrive (wrong under LATE, still right when they land at issue)."""
    def loosen(text):
        return text.replace("if constexpr (FILL) wait_vm_lgkm0<(NSTAGE - 2) * LPT>();",
                            "if constexpr (FILL) wait_vm_lgkm0<(NSTAGE - 1) * LPT>();")
    lib = _build(str(tmp_path), "emu_gemm", "gemm_harness.cpp", ["common.h", "gemm_f16_common.h", "gemm_f16_pipe.h"],
                 mutate={"gemm_f16_pipe.h": loosen}, defines=("EMU_MINIMAL", ))
    lib.emu_gemm.restype = ctypes.c_int
    for cfg in (4, 5, 7):
        assert _fails(lambda: _run_gemm(lib, cfg, 0, 0, 0, 256, 256, 576, 1, seed=3, late=1)), cfg
    _run_gemm(lib, 5, 0, 0, 0, 256, 256, 576, 1, seed=3, late=0)


def test_a_missing_barrier_is_detected(tmp_path):
    """Without the barrier of the last sub-step a wavefront that runs ahead refills a tile the others still read (or
    reads one they have not finished waiting for)."""
    def drop(text):
        i = text.index("if constexpr (FILL) wait_vm_lgkm0<(NSTAGE - 2) * LPT>();")
        j = text.index("__builtin_amdgcn_s_barrier();", i)
        return text[:j] + text[j + len("__builtin_amdgcn_s_barrier();"):]
    lib = _build(str(tmp_path), "emu_gemm", "gemm_harness.cpp", ["common.h", "gemm_f16_common.h", "gemm_f16_pipe.h"],
                 mutate={"gemm_f16_pipe.h": drop}, defines=("EMU_MINIMAL", ))
    lib.emu_gemm.restype = ctypes.c_int
    for cfg in (4, 5):
        assert _fails(lambda: _run_gemm(lib, cfg, 0, 0, 0, 256, 256, 576, 1, seed=3, late=0)), cfg


def test_a_mask_that_one_kernel_ignores_is_detected(tmp_path):
    def ignore(text):
        return text.replace("if constexpr (MASK) mask2 = (float)a.mask[b0 * a.ms[0] + b1 * a.ms[1] + krow] * kLog2eF;",
                            "if constexpr (MASK) mask2 = 0.f * (float)a.mask[0];")
    lib = _build(str(tmp_path), "emu_attention", "attention_harness.cpp", ["common.h", "attention.hip"],
                 mutate={"attention_emu.h": ignore})
    lib.emu_attention.restype = ctypes.c_int
    assert _fails(lambda: _attention_case(lib, 2, 2, 128, 128, "pad", seed=4, late=0))
    _attention_case(lib, 2, 2, 128, 128, None, seed=4, late=0)


# ----------------------------------------------------------------------------- fused attention
@pytest.fixture(scope="module")
def attention_lib(tmp_path_factory):
    lib = _build(str(tmp_path_factory.mktemp("emu_attention")), "emu_attention", "attention_harness.cpp",
                 ["common.h", "attention.hip"])
    lib.emu_attention.restype = ctypes.c_int
    return lib


def _attention_case(lib, b0, b1, sq, sk, mask_kind, seed, late):
    from daceml_amd import _lib as L
    from oracle import ops as O
    r = np.random.default_rng(50 + sq + sk)
    q, k, v, do = (r.standard_normal((b0, b1, s_, 64)).astype(np.float16) for s_ in (sq, sk, sk, sq))
    mask, m64, ms = None, None, None
    if mask_kind:
        per_head = "h" in mask_kind
        pitch = (sk + 3) // 4 * 4
        mem = np.zeros((b0, b1 if per_head else 1, 1, pitch), np.float16)
        if "pad" in mask_kind:
            for b in range(b0):
                mem[b, :, :, max(1, sk - 5 - 9 * b):sk] = -10000.0
        elif "inf" in mask_kind:
            mem[..., sk // 2:sk] = -np.inf
        else:
            mem[..., :sk] = (r.standard_normal(mem[..., :sk].shape) * 2).astype(np.float16)
        mask, m64 = mem, mem[..., :sk].astype(np.float64)
        ms = (ctypes.c_int64 * 2)(mem.shape[1] * pitch if b0 > 1 else 0, pitch if per_head and b1 > 1 else 0)
    d = L.AttentionDesc()
    d.batch[0], d.batch[1], d.seq_q, d.seq_k, d.head_dim, d.scale = b0, b1, sq, sk, 64, 0.125
    for name, s_ in (("q_stride", sq), ("k_stride", sk), ("v_stride", sk), ("o_stride", sq)):
        st = getattr(d, name)
        st[0], st[1], st[2] = b1 * s_ * 64, s_ * 64, 64
    out = np.full(q.shape, np.nan, np.float16)
    lse = np.full((b0, b1, sq), np.nan, np.float32)
    dq, dk, dv = (np.full(t.shape, np.nan, np.float16) for t in (q, k, v))
    dvec = np.full((b0, b1, sq), np.nan, np.float32)
    ptr = lambda a: None if a is None else a.ctypes.data_as(ctypes.c_void_p)  # noqa: E731
    for which in (0, 1, 2):
        status = lib.emu_attention(which, ctypes.byref(d), ptr(q), ptr(k), ptr(v), ptr(out), ptr(lse), ptr(do), ptr(dq),
                                   ptr(dk), ptr(dv), ptr(dvec), ptr(mask), ms, seed, late)
        assert status == 0, "kernel %d: status %d" % (which, status)
    f64 = lambda t: t.astype(np.float64)  # noqa: E731
    want, want_lse = O.attention(f64(q), f64(k), f64(v), 0.125, m64)
    what = "%s mask=%s seed %d %s" % ((b0, b1, sq, sk), mask_kind, seed, "late" if late else "early")
    np.testing.assert_allclose(out.astype(np.float64), want, rtol=2e-2, atol=1e-2, err_msg=what)
    np.testing.assert_allclose(lse, want_lse, rtol=1e-3, atol=1e-3, err_msg=what + " (lse)")
    # the backward kernels read the forward output as the forward kernel rounded it
    for name, got, w in zip(("dq", "dk", "dv"), (dq, dk, dv), O.attention_backward(f64(q), f64(k), f64(v), 0.125, f64(do), m64)):
        np.testing.assert_allclose(got.astype(np.float64), w, rtol=2e-2, atol=1e-2 * max(1.0, float(np.abs(w).max())),
                                   err_msg="%s %s" % (name, what))
    if mask_kind == "inf":
        assert not dk[:, :, sk // 2:].any() and not dv[:, :, sk // 2:].any()


@pytest.mark.parametrize("late", [0, 1])
def test_attention_kernels_without_a_mask(attention_lib, late):
    """The instantiations that run on hardware: the model must reproduce them before it says anything about the
    masked ones."""
    _attention_case(attention_lib, 1, 2, 128, 128, None, seed=1, late=late)
    _attention_case(attention_lib, 1, 1, 100, 77, None, seed=2, late=late)
    _attention_case(attention_lib, 1, 1, 64, 321, None, seed=3, late=late)


@pytest.mark.parametrize("late", [0, 1])
@pytest.mark.parametrize("mask_kind", ["pad", "bias", "h-bias", "inf"])
def test_attention_kernels_with_an_additive_mask(attention_lib, mask_kind, late):
    """Forward, dQ and dK / dV kernels with the mask: whole and ragged key tiles (the last tile reads the mask element
    by element), a mask shared by the heads or one per head, large negative and -inf entries."""
    _attention_case(attention_lib, 2, 2, 128, 128, mask_kind, seed=4, late=late)
    _attention_case(attention_lib, 2, 1, 100, 77, mask_kind, seed=5, late=late)
    _attention_case(attention_lib, 1, 2, 40, 200, mask_kind, seed=6, late=late)


# ----------------------------------------------------------------------------- fused pointwise + depthwise convolution
def _conv_fused_lib(tmp, mutate=None):
    lib = _build(tmp, "emu_conv_fused", "conv_fused_harness.cpp", ["common.h", "conv_geom.h", "conv_fused.hip"], mutate)
    lib.emu_expand_depthwise.restype = ctypes.c_int
    return lib


@pytest.fixture(scope="module")
def conv_fused_lib(tmp_path_factory):
    return _conv_fused_lib(str(tmp_path_factory.mktemp("emu_conv_fused")))


def _expand_depthwise_problem(n, cin, cmid, h, w, stride, acts, bias):
    from oracle import ops as O
    r = np.random.default_rng(140)
    x = r.standard_normal((n, cin, h, w)).astype(np.float32)
    w1 = (r.standard_normal((cmid, cin, 1, 1)) * np.sqrt(2.0 / cin)).astype(np.float32)
    w2 = (r.standard_normal((cmid, 1, 3, 3)) * np.sqrt(2.0 / 9)).astype(np.float32)
    b1 = (r.standard_normal(cmid) * 0.1).astype(np.float32) if bias else None
    b2 = (r.standard_normal(cmid) * 0.1).astype(np.float32) if bias else None
    f1, f2 = {0: (lambda t: t, lambda t: t), 1: (O.swish, O.swish), 2: (lambda t: np.maximum(t, 0.0), lambda t: t)}[acts]
    f64 = lambda t: None if t is None else t.astype(np.float64)  # noqa: E731
    mid = f1(O.conv2d(f64(x), f64(w1), f64(b1)))
    want = f2(O.conv2d(mid, f64(w2), f64(b2), (stride, stride), (1, 1, 1, 1), (1, 1), cmid))
    return (x, w1, b1, w2, b2), want


def _run_expand_depthwise(lib, mode, rows, waves, cus, acts, shape, operands, want, seed):
    y = np.full(want.shape, np.nan, np.float32)
    geometry = (ctypes.c_int * 4)()
    ptr = lambda a: None if a is None else a.ctypes.data_as(ctypes.c_void_p)  # noqa: E731
    status = lib.emu_expand_depthwise(mode, rows, waves, cus, acts, *shape, *[ptr(t) for t in operands], ptr(y), seed,
                                      geometry)
    what = "%s mode %d rows %d waves %d cus %d seed %d geometry %s" % (shape, mode, rows, waves, cus, seed, list(geometry))
    assert status == 0, "status %d: %s" % (status, what)
    np.testing.assert_allclose(y, want, rtol=1e-5, atol=4e-6, err_msg=what)
    return y, list(geometry)


# n, cin, cmid, h, w, stride | activations (0 none/none, 1 swish/swish, 2 relu/none), biases
EXPAND_DEPTHWISE_SHAPES = [
    ((2, 16, 32, 9, 11, 2), 1, True),        # odd sizes, stride 2, the last batch is short
    ((3, 32, 64, 14, 14, 1), 0, True),
    ((1, 48, 32, 7, 5, 1), 2, False),        # three input-channel steps, rows narrower than a tile of pixels
    ((2, 32, 64, 5, 70, 2), 0, True),        # rows wider than a wavefront
    ((1, 16, 32, 1, 1, 1), 1, True),         # a single pixel: every neighbour is padding, divisions by a width of 1
    ((1, 32, 64, 40, 40, 1), 2, False),
    ((1, 32, 32, 112, 112, 2), 1, True),     # the rows of the benchmarked MBConv block, one image, one channel block
    ((1, 16, 32, 37, 130, 1), 1, True),
]


@pytest.mark.parametrize("shape,acts,bias", EXPAND_DEPTHWISE_SHAPES)
def test_expand_depthwise_rolling_window(conv_fused_lib, shape, acts, bias):
    """The strip kernel (which runs on hardware: the model has to reproduce it) and the rolling-window kernel on the
    same problems: every batch height, 8 and 16 wavefronts, segmentations from one segment per image to one per batch
    (driven by the number of compute units the workgroups are spread over), several wavefront orders. The rolling
    kernel adds in the strip kernel's order, so the two agree bit for bit."""
    operands, want = _expand_depthwise_problem(*shape, acts, bias)
    ref, _ = _run_expand_depthwise(conv_fused_lib, 0, 2, 8, 256, acts, shape, operands, want, seed=1)
    seen = set()
    for rows, waves, cus, seed in [(0, 8, 256, 1), (1, 8, 1, 2), (2, 16, 3, 3), (4, 8, 2, 4), (2, 8, 7, 5), (0, 16, 1, 6)]:
        got, geometry = _run_expand_depthwise(conv_fused_lib, 1, rows, waves, cus, acts, shape, operands, want, seed)
        assert np.array_equal(got, ref), "rolling window differs from the strips: rows %d waves %d" % (rows, waves)
        seen.add(tuple(geometry))
    if shape[3] >= 14:
        assert len({g[3] for g in seen}) > 1 and len({g[0] for g in seen}) > 1, "one geometry only: %s" % seen


def test_rolling_window_geometry_of_the_benchmarked_block(conv_fused_lib):
    """[96,32,112,112] -> 192 channels, stride 2, on 256 compute units. The library's choice (rows 0): one output row
    per batch in a ring of five expanded rows (73 KB of LDS, so two workgroups share a compute unit); the most rows
    that fit (rows -1): two per batch in a ring of nine (137 KB)."""
    shape = (1, 32, 32, 112, 112, 2)
    operands, want = _expand_depthwise_problem(*shape, 1, True)
    # one image and one channel block of the block's 96 x 6: the same rows, spread as if over 256 / (96 * 6) of a chip
    _, geometry = _run_expand_depthwise(conv_fused_lib, 1, 0, 8, 256, 1, shape, operands, want, seed=7)
    assert geometry[:2] == [1, 5]
    _, geometry = _run_expand_depthwise(conv_fused_lib, 1, -1, 8, 256, 1, shape, operands, want, seed=7)
    assert geometry[:2] == [2, 9]


def test_a_ring_one_row_short_is_detected(tmp_path):
    """Teeth: with one row less in the ring, the rows a batch adds land on a row the running stencil still reads."""
    def shrink(text):
        return text.replace("a.ring = 2 * r * stride + 3 - stride;", "a.ring = 2 * r * stride + 2 - stride;")
    lib = _conv_fused_lib(str(tmp_path), {"conv_fused_emu.h": shrink})
    shape = (1, 16, 32, 24, 20, 1)
    operands, want = _expand_depthwise_problem(*shape, 0, True)
    failures = 0
    for seed in range(1, 7):
        try:
            _run_expand_depthwise(lib, 1, 2, 8, 1, 0, shape, operands, want, seed)
        except AssertionError:
            failures += 1
    assert failures, "no wavefront order exposed the short ring"


def test_a_missing_barrier_between_batches_is_detected(tmp_path):
    def drop(text):
        marker = "            consume(oy0, oy1, wave, WAVES);\n        }\n        __syncthreads();"
        return text.replace(marker, "            consume(oy0, oy1, wave, WAVES);\n        }")
    lib = _conv_fused_lib(str(tmp_path), {"conv_fused_emu.h": drop})
    shape = (1, 16, 32, 24, 20, 1)
    operands, want = _expand_depthwise_problem(*shape, 0, True)
    failures = 0
    for seed in range(1, 7):
        try:
            _run_expand_depthwise(lib, 1, 2, 8, 1, 0, shape, operands, want, seed)
        except AssertionError:
            failures += 1
    assert failures, "no wavefront order exposed the missing barrier"


# ----------------------------------------------------------------------------- constant pad
@pytest.fixture(scope="module")
def pad_lib(tmp_path_factory):
    lib = _build(str(tmp_path_factory.mktemp("emu_pad")), "emu_pad", "pad_harness.cpp", ["common.h", "pad.hip"])
    lib.emu_pad.restype = ctypes.c_int
    return lib


@pytest.mark.parametrize("shape,pads,value", [
    ((2, 3, 5, 7), (0, 0, 1, 2, 0, 0, 3, 0), 0.0),           # spatial axes, lopsided
    ((2, 3, 5, 7), (1, 2, 0, 0, 0, 1, 0, 0), -1.5),          # batch and channel axes, a fill value
    ((4, 9), (-1, 2, 0, -3), 7.0),                           # cropping and padding mixed
    ((3, 4, 6), (0, -1, -2, 0, -1, -1), 0.0),                # cropping only: the reverse of a pad
    ((300, 41), (2, 1, 3, 0), 0.25),                         # more than one workgroup
    ((5, ), (0, 0), 0.0),                                    # nothing to do
    ((2, 2, 2, 2, 2, 3), (1, 0, 0, 1, 0, 0, 0, 1, 0, 0, 1, 2), 1.0)])   # six axes
def test_constant_pad_kernel(pad_lib, shape, pads, value):
    """The kernel's index arithmetic, through its own host function (which also builds the launch geometry)."""
    r = np.random.default_rng(len(shape) * 10 + len(pads))
    x = r.standard_normal(shape).astype(np.float32)
    nd = len(shape)
    begin, end = pads[:nd], pads[nd:]
    crop = x[tuple(slice(max(-b, 0), d - max(-e, 0)) for d, b, e in zip(shape, begin, end))]
    want = np.pad(crop, [(max(b, 0), max(e, 0)) for b, e in zip(begin, end)], constant_values=np.float32(value))
    y = np.full(want.shape, np.nan, np.float32)
    i64 = lambda t: (ctypes.c_int64 * len(t))(*t)  # noqa: E731
    status = pad_lib.emu_pad(x.ctypes.data_as(ctypes.c_void_p), y.ctypes.data_as(ctypes.c_void_p), nd, i64(shape),
                             i64(begin), i64(end), ctypes.c_float(value), 1)
    assert status == 0
    assert np.array_equal(y, want)


def test_constant_pad_refuses_a_crop_larger_than_the_axis(pad_lib):
    x = np.zeros((4, 4), np.float32)
    i64 = lambda t: (ctypes.c_int64 * len(t))(*t)  # noqa: E731
    assert pad_lib.emu_pad(x.ctypes.data_as(ctypes.c_void_p), x.ctypes.data_as(ctypes.c_void_p), 2, i64((4, 4)),
                           i64((-3, 0)), i64((-2, 0)), ctypes.c_float(0.0), 1) < 0


# ----------------------------------------------------------------------------- MaxPool
@pytest.fixture(scope="module")
def pool_lib(tmp_path_factory):
    lib = _build(str(tmp_path_factory.mktemp("emu_pool")), "emu_pool", "pool_harness.cpp", ["common.h", "pool.hip"])
    lib.emu_maxpool.restype = ctypes.c_int
    lib.emu_maxpool.argtypes = [ctypes.c_void_p] * 3 + [ctypes.c_int64] * 7 + [ctypes.c_uint]
    return lib


@pytest.mark.parametrize("shape,kernel,stride", [((2, 6, 28, 28), (2, 2), (2, 2)),     # the pools of the reference's LeNet
                                                 ((2, 3, 13, 13), (2, 2), (2, 2)),     # a last row and column left over
                                                 ((1, 2, 9, 7), (3, 3), (2, 2)),       # overlapping windows
                                                 ((2, 1, 7, 10), (3, 2), (1, 3)),      # gaps between windows
                                                 ((1, 1, 5, 5), (5, 5), (1, 1)),       # one window
                                                 ((1, 2, 4, 4), (1, 1), (1, 1))])      # the identity
def test_maxpool_kernels(pool_lib, shape, kernel, stride):
    """Forward and backward kernels through their host functions against PyTorch (which also sends the gradient to the
    first maximum of a window); quantised inputs make equal maxima common."""
    import torch
    r = np.random.default_rng(sum(shape))
    x = np.round(r.standard_normal(shape) * 2).astype(np.float32)
    n, c, h, w = shape
    xt = torch.tensor(x.astype(np.float64), requires_grad=True)
    want = torch.nn.functional.max_pool2d(xt, kernel, stride)
    dy = r.standard_normal(tuple(want.shape)).astype(np.float32)
    want.backward(torch.tensor(dy.astype(np.float64)))
    y = np.full(tuple(want.shape), np.nan, np.float32)
    dx = np.full(shape, np.nan, np.float32)
    ptr = lambda a: a.ctypes.data_as(ctypes.c_void_p)  # noqa: E731
    assert pool_lib.emu_maxpool(ptr(x), None, ptr(y), n * c, h, w, *kernel, *stride, 1) == 0
    assert np.array_equal(y, want.detach().numpy().astype(np.float32))
    assert pool_lib.emu_maxpool(ptr(x), ptr(dy), ptr(dx), n * c, h, w, *kernel, *stride, 2) == 0
    np.testing.assert_allclose(dx, xt.grad.numpy(), rtol=1e-6, atol=1e-6)
