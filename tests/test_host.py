"""CPU-only tests of the host side: the C ABI loads and exports what include/daceml_hip.h declares,
argument errors are reported before any device work, the einsum planner, the library-node registry
(three selection levels, late registration, validation), the fusion pass and the autodiff registry."""
import ctypes
import os
import re

import numpy as np
import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


# ----------------------------------------------------------------------------- C ABI
def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "daceml_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(dmlhip_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol(lib):
    from daceml_amd import _lib as L
    names = _declared_symbols()
    assert len(names) >= 35
    for n in names:
        assert hasattr(lib, n), "libdaceml_hip.so does not export %s" % n
        assert n in L.SIGNATURES, "%s has no ctypes signature" % n
    assert sorted(L.SIGNATURES) == names
    assert lib.dmlhip_version() == 100


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    from daceml_amd import _lib as L
    monkeypatch.setattr(L, "_lib", None)
    monkeypatch.setattr(L, "LIB_PATH", str(tmp_path / "nope.so"))
    with pytest.raises(L.HipLibraryMissing):
        L.load()


def test_argument_errors_need_no_gpu(lib):
    """Negative return codes come from host-side validation, before any launch."""
    from daceml_amd import _lib as L
    p = ctypes.c_void_p(16)  # never dereferenced
    assert lib.dmlhip_softmax_f16(p, p, -1, 4, None) == L.ERR_SHAPE
    assert "negative" in L.last_error()
    assert lib.dmlhip_softmax_f16(None, p, 4, 4, None) == L.ERR_NULL
    assert lib.dmlhip_softmax_f32(None, None, 0, 16, None) == 0          # empty: no-op, not an error
    assert lib.dmlhip_layernorm_f16(p, None, p, p, p, None, None, None, 4, 8, -1.0, None) == L.ERR_SHAPE
    assert lib.dmlhip_layernorm_backward_f16(p, p, p, p, p, p, p, p, 8, 64, None, 0, None) == L.ERR_WORKSPACE
    assert lib.dmlhip_layernorm_backward_workspace_bytes(4096, 1024) > 0
    shape = L.i64_array([4, 4])
    assert lib.dmlhip_binary_f16(99, p, p, p, 2, shape, shape, shape, None) == L.ERR_ENUM
    assert lib.dmlhip_binary_f16(L.ADD, p, p, p, 9, shape, shape, shape, None) == L.ERR_SHAPE
    assert lib.dmlhip_unary_f32(L.GELU, ctypes.c_void_p(2), p, 8, 0.0, None) == L.ERR_ALIGN
    assert lib.dmlhip_cast(L.F16, 7, p, p, 4, None) == L.ERR_ENUM
    perm = L.i64_array([0, 0])
    assert lib.dmlhip_transpose_f16(p, p, 2, shape, perm, None) == L.ERR_SHAPE
    assert lib.dmlhip_reduce_f16(L.RMEAN, p, p, L.F32, 4, 0, 1, None, 0, None) == L.ERR_SHAPE   # mean of nothing
    d = L.GemmDesc()
    d.m, d.n, d.k = 4, 4, -1
    assert lib.dmlhip_gemm_f16(ctypes.byref(d), p, p, p, None, None, None, None) == L.ERR_SHAPE
    d.k = 4
    d.batch[0] = d.batch[1] = d.batch[2] = 1
    d.c_stride_m = 2  # rows of C would overlap
    assert lib.dmlhip_gemm_f16(ctypes.byref(d), p, p, p, None, None, None, None) == L.ERR_SHAPE
    d.c_stride_m = 4
    d.out_dtype = 5
    assert lib.dmlhip_gemm_f16(ctypes.byref(d), p, p, p, None, None, None, None) == L.ERR_ENUM
    d.out_dtype = L.F16
    assert lib.dmlhip_gemm_f32(ctypes.byref(d), p, p, p, None, None, None, None) == L.ERR_ENUM  # f32 in -> f32 out
    assert lib.dmlhip_gemm_f16(None, p, p, p, None, None, None, None) == L.ERR_NULL
    c = L.Conv2dDesc()
    c.n, c.c, c.h, c.w, c.m, c.kh, c.kw = 1, 4, 8, 8, 6, 3, 3
    c.stride_h = c.stride_w = c.dil_h = c.dil_w = 1
    c.group = 3   # 4 channels not divisible by 3
    assert lib.dmlhip_conv2d_f32(ctypes.byref(c), p, p, None, p, None) == L.ERR_SHAPE
    c.group = 1
    oh, ow = ctypes.c_int64(), ctypes.c_int64()
    assert lib.dmlhip_conv2d_out_shape(ctypes.byref(c), ctypes.byref(oh), ctypes.byref(ow)) == 0
    assert (oh.value, ow.value) == (6, 6)
    c.stride_h = c.stride_w = 2   # config 1 of the baseline: 10x10, k3, s2 -> 4x4
    c.h = c.w = 10
    lib.dmlhip_conv2d_out_shape(ctypes.byref(c), ctypes.byref(oh), ctypes.byref(ow))
    assert (oh.value, ow.value) == (4, 4)


def test_argument_errors_of_the_grouped_and_fused_entry_points(lib):
    """Grouped / K-summed / row-sum contractions, attention and BatchNormalization validate on the host too."""
    from daceml_amd import _lib as L
    p = ctypes.c_void_p(32)
    table = (ctypes.c_void_p * 4)(32, 32, 32, 32)
    holes = (ctypes.c_void_p * 4)(32, 0, 32, 32)
    d = L.GemmDesc()
    d.m, d.n, d.k = 128, 128, 64
    d.batch[0] = d.batch[1] = d.batch[2] = 1
    d.a_stride_m, d.a_stride_k, d.b_stride_k, d.b_stride_n, d.c_stride_m = 64, 1, 1, 64, 128
    d.alpha = 1.0
    ref = ctypes.byref(d)
    assert lib.dmlhip_gemm_f16_grouped(ref, 0, table, table, table, None, None, 0, None) == L.ERR_SHAPE
    assert lib.dmlhip_gemm_f16_grouped(ref, 5, table, table, table, None, None, 0, None) == L.ERR_SHAPE
    assert lib.dmlhip_gemm_f16_grouped(ref, 2, None, table, table, None, None, 0, None) == L.ERR_NULL
    assert lib.dmlhip_gemm_f16_grouped(ref, 3, table, table, holes, None, None, 0, None) == L.ERR_NULL
    assert lib.dmlhip_gemm_f16_ksum(ref, 5, table, table, p, None, None, None) == L.ERR_SHAPE
    assert lib.dmlhip_gemm_f16_ksum(ref, 3, table, holes, p, None, None, None) == L.ERR_NULL
    assert lib.dmlhip_gemm_f16_ksum(ref, 2, table, table, None, None, None, None) == L.ERR_NULL
    d.beta = 1.0
    assert lib.dmlhip_gemm_f16_ksum(ref, 2, table, table, p, None, None, None) == L.ERR_UNSUPPORTED
    d.beta = 0.0
    # row sums: A must be a dense [k, m] matrix, the product unbatched, the sums fp16 / fp32
    assert lib.dmlhip_gemm_f16_grouped_asum(ref, 1, table, table, table, table, L.F32, None, 0, None) == L.ERR_UNSUPPORTED
    d.a_stride_m, d.a_stride_k = 1, 128
    assert lib.dmlhip_gemm_f16_grouped_asum(ref, 1, table, table, table, table, 7, None, 0, None) == L.ERR_ENUM
    assert lib.dmlhip_gemm_f16_grouped_asum(ref, 1, table, table, table, None, L.F32, None, 0, None) == L.ERR_NULL
    d.batch[1] = 2
    assert lib.dmlhip_gemm_f16_grouped_asum(ref, 1, table, table, table, table, L.F32, None, 0, None) == L.ERR_SHAPE
    d.batch[1] = 1
    assert lib.dmlhip_gemm_f16_grouped_asum_workspace_bytes(ref) >= 0
    a = L.AttentionDesc()
    a.batch[0], a.batch[1], a.seq_q, a.seq_k, a.head_dim = 1, 2, 64, 64, 64
    for arr in (a.q_stride, a.k_stride, a.v_stride, a.o_stride):
        arr[0], arr[1], arr[2] = 2 * 64 * 64, 64 * 64, 64
    a.scale = 0.125
    assert lib.dmlhip_attention_f16(ctypes.byref(a), p, p, None, p, None, None) == L.ERR_NULL
    a.scale = -1.0
    assert lib.dmlhip_attention_f16(ctypes.byref(a), p, p, p, p, None, None) == L.ERR_SHAPE
    assert "scale" in L.last_error()
    a.scale, a.head_dim = 0.125, 32
    assert lib.dmlhip_attention_f16(ctypes.byref(a), p, p, p, p, None, None) == L.ERR_UNSUPPORTED
    assert lib.dmlhip_batchnorm_inference_f32(p, p, p, p, p, p, 2, 0, 16, 1e-5, None) == L.ERR_SHAPE
    assert lib.dmlhip_batchnorm_training_f16(p, p, p, p, p, p, p, p, p, p, 2, 3, 16, 1e-5, 0.9, None, 0, None) == \
        L.ERR_WORKSPACE
    assert lib.dmlhip_batchnorm_backward_f32(p, p, p, p, p, None, None, None, 2, 3, 16, 1e-5, p, 1 << 20, None) == L.ERR_NULL
    assert lib.dmlhip_batchnorm_workspace_bytes(8, 3, 1024) > 0
    # pointwise + depthwise in one kernel: the pair of descriptors must describe that chain
    pw, dw = L.Conv2dDesc(), L.Conv2dDesc()
    pw.n, pw.c, pw.h, pw.w, pw.m, pw.kh, pw.kw = 2, 16, 8, 8, 32, 1, 1
    pw.stride_h = pw.stride_w = pw.dil_h = pw.dil_w = pw.group = 1
    dw.n, dw.c, dw.h, dw.w, dw.m, dw.kh, dw.kw = 2, 32, 8, 8, 32, 3, 3
    dw.stride_h = dw.stride_w = dw.pad_h = dw.pad_w = dw.dil_h = dw.dil_w = 1
    dw.group = 32
    fused = lambda *a: lib.dmlhip_conv2d_expand_depthwise_f32(ctypes.byref(pw), ctypes.byref(dw), *a)
    assert fused(p, p, None, None, None, p, None) == L.ERR_NULL
    dw.stride_h = dw.stride_w = 3
    assert fused(p, p, None, p, None, p, None) == L.ERR_UNSUPPORTED
    dw.stride_h = dw.stride_w = 1
    dw.h = 9
    assert fused(p, p, None, p, None, p, None) == L.ERR_SHAPE
    dw.h = 8
    pw.c = 8
    assert fused(p, p, None, p, None, p, None) == L.ERR_UNSUPPORTED
    pw.c = 16
    pw.act = L.ACT_GELU
    assert fused(p, p, None, p, None, p, None) == L.ERR_ENUM


def test_kernels_refuse_host_tensors():
    from daceml_amd import kernels as K
    with pytest.raises(ValueError):
        K.softmax(torch.zeros(2, 4, dtype=torch.float16))
    with pytest.raises(TypeError):
        K._fn("softmax", torch.float64)


# ----------------------------------------------------------------------------- einsum planner
def _plan(eq, sa, sb, stra=None, strb=None):
    from daceml_amd import contraction as C
    return C.plan_contraction(eq, sa, stra or C.contiguous_strides(sa), sb, strb or C.contiguous_strides(sb))


def test_planner_bert_contractions():
    from daceml_amd import contraction as C
    p = _plan("aik,kj->aij", (8, 512, 1024), (1024, 1024))
    assert (p.m, p.n, p.k, p.batch) == (4096, 1024, 1024, [1, 1, 1]) and p.a_stride_k == 1 and p.b_stride_n == 1
    p = _plan("aik,jk->aij", (8, 512, 1024), (4096, 1024))          # weight stored [out, in]
    assert (p.b_stride_k, p.b_stride_n) == (1, 1024)
    p = _plan("baik,bakj->baij", (8, 16, 512, 64), (8, 16, 64, 512))
    assert (p.m, p.n, p.k, p.batch) == (512, 512, 64, [1, 1, 128])
    p = _plan("biak,bjak->baij", (8, 512, 16, 64), (8, 512, 16, 64))  # head split folded into strides
    assert p.batch == [1, 8, 16] and p.a_stride_m == 1024 and p.a_stride_batch[1:] == [512 * 1024, 64]
    p = _plan("baik,bkaj->biaj", (8, 16, 512, 512), (8, 512, 16, 64))  # head merge folded into C's strides
    assert p.n == 64 and p.c_stride_m == 1024 and p.c_stride_batch[1:] == [512 * 1024, 64]
    p = _plan("aij,aik->jk", (8, 512, 4096), (8, 512, 1024))        # weight gradient: K = (a, i) merged
    assert (p.m, p.n, p.k) == (4096, 1024, 4096) and p.a_stride_m == 1 and not p.swapped
    p = _plan("ik,kj->ji", (4, 5), (5, 6))
    assert p.swapped and (p.m, p.n) == (6, 4)
    assert p.flops == 2 * 4 * 5 * 6
    assert C.reverse_equation("ik,kj->ij", 0) == ([1], "ij,kj->ik")
    assert C.reverse_equation("ik,kj->ij", 1) == ([0], "ij,ik->kj")
    assert C.matmul_equation(3, 2) == "aik,kj->aij" and C.matmul_equation(4, 4) == "baik,bakj->baij"
    assert C.transpose_perm("zyxw->zxyw") == [0, 2, 1, 3] and C.transpose_perm("ij->i") is None


@pytest.mark.parametrize("eq,sa,sb", [("ii,ij->j", (3, 3), (3, 4)), ("ij,jk->ik...", (2, 2), (2, 2)),
                                      ("ijl,jk->ik", (2, 3, 4), (3, 5)), ("bik,bkj->ijb", (2, 3, 4), (2, 4, 5))])
def test_planner_refuses(eq, sa, sb):
    from daceml_amd import contraction as C
    with pytest.raises(C.NotApplicable):
        _plan(eq, sa, sb)


def test_planner_matches_numpy_semantics_by_emulation():
    """Execute plans with plain index arithmetic on the host: pins the stride bookkeeping."""
    from daceml_amd import contraction as C
    rng = np.random.default_rng(0)
    for eq, sa, sb in [("biak,bjak->baij", (2, 5, 3, 4), (2, 6, 3, 4)), ("aij,aik->jk", (2, 3, 4), (2, 3, 5)),
                       ("ik,kj->ji", (3, 4), (4, 5)), ("baik,bkaj->biaj", (2, 3, 4, 5), (2, 5, 3, 6))]:
        a, b = rng.standard_normal(sa), rng.standard_normal(sb)
        p = _plan(eq, sa, sb)
        x, y = (b, a) if p.swapped else (a, b)
        xf, yf = x.reshape(-1), y.reshape(-1)
        out = np.zeros(int(np.prod(p.out_shape)))
        for z0 in range(p.batch[0]):
            for z1 in range(p.batch[1]):
                for z2 in range(p.batch[2]):
                    z = (z0, z1, z2)
                    ao = sum(z[i] * p.a_stride_batch[i] for i in range(3))
                    bo = sum(z[i] * p.b_stride_batch[i] for i in range(3))
                    co = sum(z[i] * p.c_stride_batch[i] for i in range(3))
                    for m in range(p.m):
                        for n in range(p.n):
                            acc = 0.0
                            for k in range(p.k):
                                acc += xf[ao + m * p.a_stride_m + k * p.a_stride_k] * \
                                       yf[bo + k * p.b_stride_k + n * p.b_stride_n]
                            out[co + m * p.c_stride_m + n] = acc
        np.testing.assert_allclose(out.reshape(p.out_shape), np.einsum(eq, a, b), rtol=1e-12)


# ----------------------------------------------------------------------------- registry
def _softmax_sdfg(dtype=torch.float16, shape=(4, 8)):
    import daceml_amd.onnx as donnx
    from daceml_amd.sdfg import SDFG
    sdfg = SDFG("t")
    st = sdfg.add_state()
    sdfg.add_array("a", shape, dtype)
    sdfg.add_array("b", shape, dtype)
    node = donnx.ONNXSoftmax("sm", axis=-1)
    st.add_edge(st.add_read("a"), None, node, "input", sdfg.make_array_memlet("a"))
    st.add_edge(node, "output", st.add_write("b"), None, sdfg.make_array_memlet("b"))
    return sdfg, st, node


def test_registry_mirrors_reference_api():
    import daceml_amd.onnx as donnx
    from daceml_amd.onnx import ONNXForward, op_implementation
    for op in ["MatMul", "Einsum", "Gemm", "Softmax", "Add", "Sub", "Mul", "Div", "Sum", "Erf", "ReduceMean",
               "ReduceSum", "Transpose", "Conv", "GlobalAveragePool", "Sigmoid", "LayerNormalization", "Gelu",
               "BiasGelu"]:
        impls = dict(ONNXForward.registered_implementations(op))
        assert "hip" in impls, op
        assert "hip" in donnx.get_onnx_node(op).implementations
    assert donnx.has_onnx_node("Conv") and not donnx.has_onnx_node("NoSuchOp")
    with pytest.raises(ValueError):
        donnx.get_onnx_node("NoSuchOp")
    with pytest.raises(ValueError):
        donnx.ONNXEinsum("e")                     # required attribute missing
    with pytest.raises(TypeError):
        donnx.ONNXSoftmax("s", nonsense=1)

    # an implementation registered late is visible on the node class too
    calls = []

    @op_implementation(op="Softmax", name="probe")
    class Probe(ONNXForward):
        @staticmethod
        def forward_can_be_applied(node, state, sdfg):
            return sdfg.arrays["a"].dtype == torch.float16

        @staticmethod
        def forward(node, state, sdfg):
            calls.append(node.label)
            return donnx.ONNXSoftmax.implementations["hip"].forward(node, state, sdfg)

    try:
        assert "probe" in donnx.ONNXSoftmax.implementations
        # package default < class default < node.implementation
        sdfg, st, node = _softmax_sdfg()
        assert node.selected_implementation() == "hip"
        old = donnx.default_implementation
        donnx.default_implementation = "probe"
        assert node.selected_implementation() == "probe"
        donnx.ONNXSoftmax.default_implementation = "hip"
        assert node.selected_implementation() == "hip"
        node.implementation = "probe"
        assert node.selected_implementation() == "probe"
        node.expand(sdfg, st)
        assert calls == ["sm"]
        # inapplicable -> explicit refusal, no silent fallback
        sdfg32, st32, node32 = _softmax_sdfg(torch.float32)
        node32.implementation = "probe"
        with pytest.raises(donnx.NotApplicable):
            node32.expand(sdfg32, st32)
    finally:
        donnx.default_implementation = old
        donnx.ONNXSoftmax.default_implementation = None
        donnx.ONNXSoftmax.implementations.pop("probe", None)
        ONNXForward.unregister(Probe)


def test_validate_checks_connectors():
    import daceml_amd.onnx as donnx
    from daceml_amd.sdfg import SDFG
    sdfg, st, node = _softmax_sdfg()
    node.validate(sdfg, st)
    # missing required output
    sdfg2 = SDFG("v")
    st2 = sdfg2.add_state()
    sdfg2.add_array("a", (2, 2), torch.float32)
    n2 = donnx.ONNXSoftmax("s")
    st2.add_edge(st2.add_read("a"), None, n2, "input", sdfg2.make_array_memlet("a"))
    with pytest.raises(ValueError, match="output"):
        n2.validate(sdfg2, st2)
    # variadic numbering must be 0..n-1
    sdfg2.add_array("o", (2, 2), torch.float32)
    s = donnx.ONNXSum("sum")
    s.add_in_connector("data_0__1")
    st2.add_edge(st2.add_read("a"), None, s, "data_0__1", sdfg2.make_array_memlet("a"))
    st2.add_edge(s, "sum", st2.add_write("o"), None, sdfg2.make_array_memlet("o"))
    with pytest.raises(ValueError, match="numbered"):
        s.validate(sdfg2, st2)
    with pytest.raises(ValueError):
        donnx.parse_variadic_param("x__01")
    assert donnx.parse_variadic_param("Inputs__3") == ("Inputs", 3)
    # integer tensors are not supported element types
    sdfg3 = SDFG("i")
    st3 = sdfg3.add_state()
    sdfg3.add_array("a", (2, ), torch.uint8)
    sdfg3.add_array("b", (2, ), torch.uint8)
    r = donnx.ONNXRelu("r")
    st3.add_edge(st3.add_read("a"), None, r, "X", sdfg3.make_array_memlet("a"))
    st3.add_edge(r, "Y", st3.add_write("b"), None, sdfg3.make_array_memlet("b"))
    with pytest.raises(TypeError):
        r.validate(sdfg3, st3)


def test_forward_can_be_applied_never_raises_and_refuses():
    import daceml_amd.onnx as donnx
    from daceml_amd.sdfg import SDFG
    hip = donnx.ONNXConv.implementations["hip"]
    sdfg = SDFG("c")
    st = sdfg.add_state()
    sdfg.add_array("x", (1, 3, 8, 8), torch.float32)
    sdfg.add_array("w", (4, 3, 3, 3), torch.float32)
    sdfg.add_array("y", (1, 4, 6, 6), torch.float32)
    conv = donnx.ONNXConv("conv", pads=[1, 0, 0, 0])            # asymmetric pads: refused
    for arr, conn in (("x", "X"), ("w", "W")):
        st.add_edge(st.add_read(arr), None, conv, conn, sdfg.make_array_memlet(arr))
    st.add_edge(conv, "Y", st.add_write("y"), None, sdfg.make_array_memlet("y"))
    assert hip.forward_can_be_applied(conv, st, sdfg) is False
    conv.pads = None
    assert hip.forward_can_be_applied(conv, st, sdfg) is True
    conv.auto_pad = "SAME_UPPER"
    assert hip.forward_can_be_applied(conv, st, sdfg) is False
    # a node with no edges at all: False, not an exception
    assert donnx.ONNXSoftmax.implementations["hip"].forward_can_be_applied(donnx.ONNXSoftmax("s"), st, sdfg) is False
    # Einsum with an ellipsis (refused by PureEinsum as well)
    es = donnx.ONNXEinsum("e", equation="...ij,jk->...ik")
    assert donnx.ONNXEinsum.implementations["hip"].forward_can_be_applied(es, st, sdfg) is False


# ----------------------------------------------------------------------------- fusion / autodiff
def test_fusion_pipeline_on_bert_layer():
    from daceml_amd import graphs
    from daceml_amd.transformation import fusion
    sdfg = graphs.bert_encoder_layer(2, 64, 128, 4, 512, torch.float16)
    st = sdfg.states()[0]
    before = [n.schema.name for n in st.library_nodes()]
    assert before.count("MatMul") == 8 and before.count("Erf") == 1 and before.count("ReduceMean") == 4
    stats = fusion.auto_optimize(sdfg, training=True, gelu_epilogue=True)
    assert stats == {"gelu": 1, "layernorm": 2, "swish": 0, "pad_into_conv": 0, "conv_activation": 0, "batchnorm_activation": 0, "gated_conv": 0, "expand_depthwise": 0,
                     "matmul_to_einsum": 8,
                     "views": 15, "epilogues": 7, "skip_layernorm": 0, "attention": 0,   # head dim 32: not fused
                     "grouped_einsums": 0}                                               # training: after autodiff
    after = {n.label: n for n in st.library_nodes()}
    assert sorted(n.schema.name for n in after.values()) == ["Einsum"] + ["FusedEinsum"] * 7 + \
        ["LayerNormalization"] * 2 + ["Softmax"]
    assert after["scores_fused"].equation == "biak,bjak->baij"          # head split folded into letters
    assert abs(after["scores_fused"].alpha - 1 / np.sqrt(32)) < 1e-12   # Div(sqrt d) -> alpha
    assert after["context"].equation == "baik,bkaj->biaj"               # head merge folded into the output
    assert after["ffn1_matmul_fused"].activation == "gelu"
    conns = {e.dst_conn for e in st.in_edges(after["o_matmul_fused"])}
    assert conns == {"Inputs__0", "Inputs__1", "Bias", "Residual"}
    assert after["ln1_fused"].epsilon == 1e-12                          # not the fp16-rounded 0.0
    assert all(e.dst_conn != "Inputs__1" or sdfg.arrays[e.data.data].shape == (128, 128)
               for e in st.in_edges(after["q_matmul_fused"]))           # weight used as stored, no Transpose
    # an inference graph also gets its three projections grouped into one launch
    inf = graphs.bert_encoder_layer(2, 64, 128, 4, 512, torch.float16)
    assert fusion.auto_optimize(inf)["grouped_einsums"] == 2
    assert "grouped_k_q_v" in {n.label for n in inf.states()[0].library_nodes()}


def _out(state, node, conn):
    return next(iter(state.out_edges_by_connector(node, conn))).data.data


def test_attention_fusion_roles_and_graph():
    from daceml_amd import graphs
    from daceml_amd.autodiff import add_backward_pass
    from daceml_amd.transformation import fusion
    roles = fusion._attention_roles
    # BERT's head-split letters: tensors are [batch, seq, head, d]
    assert roles("biak,bjak->baij", "baik,bkaj->biaj") == (True, (0, 2, 1, 3), (0, 2, 1, 3), (0, 2, 1, 3), (0, 2, 1, 3))
    # dense [b, h, s, d]; keys given first; one batch dim; none
    assert roles("abik,abjk->abij", "abij,abjd->abid") == (True, (0, 1, 2, 3), (0, 1, 2, 3), (0, 1, 2, 3), (0, 1, 2, 3))
    assert roles("abjk,abik->abij", "abij,abjd->abid")[0] is False
    assert roles("bik,bjk->bij", "bij,bjd->bid") == (True, (-1, 0, 1, 2), (-1, 0, 1, 2), (-1, 0, 1, 2), (-1, 0, 1, 2))
    assert roles("ik,jk->ij", "ij,jd->id")[1] == (-1, -1, 0, 1)
    # not attention: softmax axis is not the contracted one of the second product; outer product; 3 batch dims
    assert roles("abik,abjk->abij", "abij,abid->abjd") is None
    assert roles("abik,abjk->abji", "abij,abjd->abid") is None or roles("abik,abjk->abji", "abij,abjd->abid")[0] is False
    assert roles("abcik,abcjk->abcij", "abcij,abcjd->abcid") is None
    assert roles("abik,abjl->abij", "abij,abjd->abid") is None

    sdfg = graphs.bert_encoder_layer(2, 64, 256, 4, 512, torch.float16)   # head dim 64
    stats = fusion.auto_optimize(sdfg, training=True)
    assert stats["attention"] == 1
    st = sdfg.states()[0]
    names = sorted(n.schema.name for n in st.library_nodes())
    # (by default the Gelu stays a node of its own: see auto_optimize)
    assert names == ["FusedAttention"] + ["FusedEinsum"] * 6 + ["Gelu"] + ["LayerNormalization"] * 2
    att = [n for n in st.library_nodes() if n.schema.name == "FusedAttention"][0]
    assert att.scale == 0.125 and att.q_perm == (0, 2, 1, 3)
    assert not any("scores" in a or "softmax" in a for a in sdfg.arrays)   # the score matrix is gone
    from oracle import bert_layer as OB
    add_backward_pass(sdfg, st, ["y"], ["x"] + OB.PARAM_NAMES)
    back = [n for n in sdfg.states()[1].library_nodes() if n.schema.name == "FusedAttentionGrad"]
    assert len(back) == 1
    ins = {e.dst_conn for e in sdfg.states()[1].in_edges(back[0])}
    assert ins == {"Q", "K", "V", "O", "LogSumExp", "dO"}
    # the six bias gradients become one node; nothing else in the state changes
    n_before = len(sdfg.states()[1].library_nodes())
    assert fusion.optimize_backward(sdfg) == {"bias_gradients": 6, "mul_reductions": 0, "row_affine": 0, "reductions": 0,
                                             "einsum_sums": 6, "grouped_einsums": 5}
    bnodes = sdfg.states()[1].library_nodes()
    # six bias-gradient reductions (now InputSum outputs of the weight-gradient contractions), two gradient sums and five
    # contractions fewer (q/k/v input gradients: 3 -> 1 EinsumSum that also adds the residual path; o/q/k/v weight
    # gradients: 4 -> 1; the other Sum rides on a contraction as its Residual)
    assert len(bnodes) == n_before - 13 and not any(n.schema.name in ("ReduceSum", "MultiReduceSum", "Sum") for n in bnodes)
    wg = [n for n in bnodes if n.schema.name == "GroupedEinsum"]
    assert len(wg) == 1 and {_out(sdfg.states()[1], wg[0], "InputSum__%d" % i) for i in range(4)} == \
        {"gradient_%s_b" % p for p in "koqv"}
    es = [n for n in bnodes if n.schema.name == "EinsumSum"]
    assert len(es) == 1 and es[0].label == "sum_k_grad_0_q_grad_0_v_grad_0"
    assert _out(sdfg.states()[1], es[0], "Output") == "gradient_x"
    assert {e.dst_conn for e in sdfg.states()[1].in_edges(es[0])} == {"A__0", "B__0", "A__1", "B__1", "A__2", "B__2", "Residual"}
    grouped = sorted(n.label for st_ in sdfg.states() for n in st_.library_nodes() if n.schema.name == "GroupedEinsum")
    assert grouped == ["grouped_k_grad_1_o_grad_1_q_grad_1_v_grad_1", "grouped_k_q_v"]
    # grouping respects data dependences, also through views: o's input gradient feeds the attention backward
    # whose outputs the q/k/v gradients read, so it stays on its own; the states still sort topologically
    assert any(n.label == "o_matmul_fused_grad_0" for n in bnodes)
    for st_ in sdfg.states():
        st_.topological_sort()
    sums = sorted(e.data.data for n in bnodes for e in sdfg.states()[1].out_edges(n) if e.src_conn.startswith("InputSum"))
    assert sums == sorted("gradient_%s_b" % p for p in ("q", "k", "v", "o", "ffn1", "ffn2"))
    # without the contraction route the six reductions still merge into one MultiReduceSum
    s2 = graphs.bert_encoder_layer(2, 64, 256, 4, 512, torch.float16)
    fusion.auto_optimize(s2, training=True)
    add_backward_pass(s2, s2.states()[0], ["y"], ["x"] + OB.PARAM_NAMES,
                      grad_dtypes={n: torch.float32 for n in OB.PARAM_NAMES})
    assert fusion.fuse_reductions(s2) == 5
    multi = [n for n in s2.states()[1].library_nodes() if n.schema.name == "MultiReduceSum"][0]
    outs = sorted(e.data.data for e in s2.states()[1].out_edges(multi))
    assert outs == sorted("gradient_%s_b" % p for p in ("q", "k", "v", "o", "ffn1", "ffn2"))
    # the forward node now also emits the log-sum-exp rows
    assert "LogSumExp" in {e.src_conn for e in st.out_edges(att)}
    # fp32 graphs keep the unfused chain (the kernel is fp16 only)
    s32 = graphs.bert_encoder_layer(2, 64, 256, 4, 512, torch.float32)
    assert fusion.auto_optimize(s32)["attention"] == 0


def test_batchnorm_activation_fusion_keeps_the_backward_pass():
    """BatchNormalization -> Sigmoid, Mul (the exporter's swish) becomes one node with the activation inside, in
    training graphs too: the gradient node then gets the activation and the bias."""
    from daceml_amd import graphs
    from daceml_amd.autodiff import add_backward_pass
    from daceml_amd.transformation import fusion
    g = graphs.GraphBuilder("bn_swish", torch.float32)
    x = g.input("x", (4, 6, 8, 8))
    for name in ("scale", "bias", "mean", "var"):
        g.input(name, (6, ))
    outs = g.node("BatchNormalization", {"X": x, "scale": "scale", "B": "bias", "in_mean": "mean", "in_var": "var"},
                  {"Y": (4, 6, 8, 8), "out_mean": (6, ), "out_var": (6, ), "saved_mean": (6, ), "saved_var": (6, )},
                  label="bn", epsilon=1e-5, momentum=0.9)
    g.output(g.swish(outs["Y"], "act"), "y")
    stats = fusion.auto_optimize(g.sdfg, training=True)
    assert stats["swish"] == 1 and stats["batchnorm_activation"] == 1
    nodes = g.state.library_nodes()
    assert [n.schema.name for n in nodes] == ["BatchNormalization"] and nodes[0]._activation == "swish"
    assert add_backward_pass(g.sdfg, g.state, ["y"], ["x", "scale", "bias"]) == \
        {"x": "gradient_x", "scale": "gradient_scale", "bias": "gradient_bias"}
    grad = [n for n in g.sdfg.states()[1].library_nodes() if n.schema.name == "BatchNormalizationGrad"]
    assert len(grad) == 1 and grad[0].activation == "swish" and "B" in grad[0].in_connectors
    assert [n.schema.name for n in g.sdfg.states()[1].library_nodes()] == ["BatchNormalizationGrad"]


def test_mul_reduce_fusion_on_a_gate_gradient():
    """y = x * gate[n, c, 1, 1]: the gate's gradient is ReduceSum(Mul(dy, x)) over the two trailing axes; after
    optimize_backward it is one MulReduceSum and the product array is gone."""
    from daceml_amd import graphs
    from daceml_amd.autodiff import add_backward_pass
    from daceml_amd.transformation import fusion
    g = graphs.GraphBuilder("gate", torch.float32)
    x, gate = g.input("x", (2, 6, 8, 8)), g.input("gate", (2, 6, 1, 1))
    g.output(g.node("Mul", {"A": x, "B": gate}, {"C": (2, 6, 8, 8)}, label="m")["C"], "y")
    add_backward_pass(g.sdfg, g.state, ["y"], ["x", "gate"])
    before = sorted(n.schema.name for n in g.sdfg.states()[1].library_nodes())
    assert before == ["Mul", "Mul", "ReduceSum"]
    assert fusion.optimize_backward(g.sdfg)["mul_reductions"] == 1
    after = {n.schema.name: n for n in g.sdfg.states()[1].library_nodes()}
    assert sorted(after) == ["Mul", "MulReduceSum"]
    assert list(after["MulReduceSum"].axes) == [2, 3] and after["MulReduceSum"].keepdims == 1
    assert not any(name.endswith("_full_B") for name in g.sdfg.arrays)      # the product array was dropped


def test_pow_backward_needs_a_constant_exponent():
    """X ** p reverses to dZ * p * X ** (p - 1) for a scalar constant p (p = 2: no Pow node left); an exponent that is
    a run-time tensor has no backward and the generator says so."""
    from daceml_amd import graphs
    from daceml_amd.autodiff import add_backward_pass
    from daceml_amd.autodiff.base_abc import AutoDiffException

    def build(exponent):
        g = graphs.GraphBuilder("pow", torch.float32)
        x = g.input("x", (4, 8))
        e = g.input("e", (4, 8)) if exponent is None else g.constant("e", exponent)
        g.output(g.node("Pow", {"X": x, "Y": e}, {"Z": (4, 8)}, label="p")["Z"], "y")
        return g

    g = build(3.0)
    assert add_backward_pass(g.sdfg, g.state, ["y"], ["x"]) == {"x": "gradient_x"}
    assert sorted(n.schema.name for n in g.sdfg.states()[1].library_nodes()) == ["Mul", "Mul", "Pow"]
    assert g.sdfg.constants_exact["p_backward_exponent"] == 2.0 and g.sdfg.constants_exact["p_backward_factor"] == 3.0
    g = build(2.0)
    add_backward_pass(g.sdfg, g.state, ["y"], ["x"])
    assert sorted(n.schema.name for n in g.sdfg.states()[1].library_nodes()) == ["Mul", "Mul"]
    g = build(None)
    with pytest.raises(AutoDiffException):
        add_backward_pass(g.sdfg, g.state, ["y"], ["x"])


def test_training_graphs_keep_differentiable_nodes():
    """Conv + activation stays two nodes when a backward pass is to come (ConvGrad differentiates a plain Conv), and
    the backward pass then builds."""
    from daceml_amd import graphs
    from daceml_amd.autodiff import add_backward_pass
    from daceml_amd.transformation import fusion

    def build():
        g = graphs.GraphBuilder("convnet", torch.float32)
        x = g.input("x", (2, 3, 8, 8))
        g.input("w", (4, 3, 3, 3))
        g.input("b", (4, ))
        y = g.node("Conv", {"X": x, "W": "w", "B": "b"}, {"Y": (2, 4, 6, 6)}, label="conv", kernel_shape=[3, 3])["Y"]
        r = g.node("Relu", {"X": y}, {"Y": (2, 4, 6, 6)}, label="relu")["Y"]
        g.output(r, "y")
        return g

    g = build()
    assert fusion.auto_optimize(g.sdfg, training=False)["conv_activation"] == 1

    # pointwise + swish + depthwise + swish -> one node, in forward graphs only and only in the kernel's tiling
    def block(cin):
        return graphs.mbconv_block(2, cin, 32, expand=6, cout=24, se_reduce=4, stride=2, dtype=torch.float32)
    sdfg = block(16)
    assert fusion.auto_optimize(sdfg)["expand_depthwise"] == 1
    fused = [n for n in sdfg.states()[0].library_nodes() if n.schema.name == "ExpandDepthwiseConv"]
    assert len(fused) == 1 and (fused[0].act_pw, fused[0].act_dw, list(fused[0].strides)) == ("swish", "swish", [2, 2])
    assert sorted(fused[0].in_connectors) == ["B_dw", "B_pw", "W_dw", "W_pw", "X"]
    assert [n.schema.name for n in sdfg.states()[0].library_nodes()].count("Conv") == 2   # the squeeze-excite pair
    assert fusion.auto_optimize(block(16), training=True)["expand_depthwise"] == 0
    assert fusion.auto_optimize(block(24))["expand_depthwise"] == 0                      # 24 input channels: not tiled
    g = build()
    assert fusion.auto_optimize(g.sdfg, training=True)["conv_activation"] == 0
    grads = add_backward_pass(g.sdfg, g.state, ["y"], ["x", "w", "b"])
    assert grads == {"x": "gradient_x", "w": "gradient_w", "b": "gradient_b"}
    assert sorted(n.schema.name for n in g.sdfg.states()[1].library_nodes()) == ["ConvGrad", "ReluGrad"]


def test_fusion_leaves_non_matching_chains_alone():
    from daceml_amd import graphs
    from daceml_amd.transformation import fusion
    g = graphs.GraphBuilder("t", torch.float32)
    x = g.input("x", (4, 8))
    y = g.gelu(x, "g")
    # a second consumer of an internal value makes the chain non-fusable
    erf_out = [a for a in g.sdfg.arrays if "erf" in a][0]
    z = g.node("Relu", {"X": erf_out}, {"Y": (4, 8)})["Y"]
    g.output(y, "y")
    g.output(z, "z")
    assert fusion.fuse_gelu(g.sdfg) == 0


def test_backward_pass_structure():
    from daceml_amd import graphs
    from daceml_amd.autodiff import (BackwardImplementation, add_backward_pass, find_backward_implementation)
    from daceml_amd.transformation import fusion
    from oracle.bert_layer import PARAM_NAMES
    sdfg = graphs.bert_encoder_layer(2, 64, 128, 4, 512, torch.float16)
    fusion.auto_optimize(sdfg, training=True, gelu_epilogue=True)
    st = sdfg.states()[0]
    grads = add_backward_pass(sdfg, st, ["y"], ["x"] + PARAM_NAMES, grad_dtypes={n: torch.float32 for n in PARAM_NAMES})
    assert grads["x"] == "gradient_x" and all(grads[n] == "gradient_" + n for n in PARAM_NAMES)
    assert sdfg.arrays["gradient_q_w"].dtype == torch.float32 and not sdfg.arrays["gradient_q_w"].transient
    assert sdfg.arrays["gradient_x"].dtype == torch.float16
    bst = sdfg.states()[1]
    names = [n.schema.name for n in bst.library_nodes()]
    assert names.count("FusedEinsum") == 16 and names.count("LayerNormalizationGrad") == 2
    assert names.count("SoftmaxGrad") == 1 and names.count("GeluGrad") == 1 and names.count("Sum") == 2
    assert names.count("ReduceSum") == 6
    # equations follow reverse_einsum_wrt_input
    eqs = {n.label: n.equation for n in bst.library_nodes() if n.schema.name == "FusedEinsum"}
    assert eqs["q_matmul_fused_grad_0"] == "aij,jk->aik" and eqs["q_matmul_fused_grad_1"] == "aij,aik->jk"
    # the forward LayerNorm nodes were given statistics outputs for the backward to read
    ln = [n for n in st.library_nodes() if n.schema.name == "LayerNormalization"][0]
    assert {e.src_conn for e in st.out_edges(ln)} == {"Y", "Mean", "InvStdDev"}
    # registry lookup honours node.backward_implementation
    sm = [n for n in st.library_nodes() if n.schema.name == "Softmax"][0]
    impl = find_backward_implementation(sdfg, st, sm)
    assert impl is not None and issubclass(impl, BackwardImplementation)
    # everything in both states expands with the hip implementations
    from daceml_amd.runtime import expand_onnx_nodes
    assert expand_onnx_nodes(sdfg) == len(names) + 11


def test_an_output_that_another_node_reads_keeps_its_incoming_gradient():
    """y0 = f(x), y1 = g(y0), both outputs: the caller's gradient of y0 is one contribution and g's reverse node
    the other; they are summed into a transient (the caller's buffer is only read), and f's reverse node reads
    that sum (accumulation rule of backward_pass_generator.py:715-752)."""
    from daceml_amd import graphs
    from daceml_amd.autodiff import add_backward_pass
    g = graphs.GraphBuilder("chain", torch.float32)
    x = g.input("x", (4, 8))
    t = g.node("Sigmoid", {"X": x}, {"Y": (4, 8)}, label="t")["Y"]
    s = g.node("Sigmoid", {"X": t}, {"Y": (4, 8)}, label="s")["Y"]
    g.output(t, "y0")
    g.output(s, "y1")
    grads = add_backward_pass(g.sdfg, g.state, ["y0", "y1"], ["x"])
    assert grads == {"x": "gradient_x"}
    bst = g.sdfg.states()[1]
    sums = [n for n in bst.library_nodes() if n.schema.name == "Sum"]
    assert len(sums) == 1
    summed = sorted(e.data.data for e in bst.in_edges(sums[0]))
    assert "gradient_y0" in summed and len(summed) == 2
    total = next(iter(bst.out_edges(sums[0]))).data.data
    assert total != "gradient_y0" and g.sdfg.arrays[total].transient
    # nothing writes the buffers the caller handed in
    written = {e.data.data for n in bst.library_nodes() for e in bst.out_edges(n)}
    assert not written & {"gradient_y0", "gradient_y1"}
    # the reverse node of the first Sigmoid reads the sum
    reads = {e.data.data for n in bst.library_nodes() if n.schema.name == "SigmoidGrad" for e in bst.in_edges(n)}
    assert total in reads


def test_expand_depthwise_fusion_asks_the_library_whether_a_strip_fits(lib):
    """The fusion pass fuses pointwise + depthwise only where the kernel's smallest row strip fits LDS, weight block
    included: a wide input-channel count that the kernel would refuse at launch stays two convolutions."""
    from daceml_amd import graphs
    from daceml_amd.transformation import fusion
    q = lib.dmlhip_conv2d_expand_depthwise_lds_bytes
    # three padded rows of 32 channels + the 32 x (Cin + 1) weight block + taps and biases, in floats
    assert q(112, 32, 2) == (32 * 3 * 114 + 32 * 33 + 320) * 4
    assert q(112, 32, 1) == q(112, 32, 2)
    assert q(112, 1024, 2) == 0 and q(5000, 32, 1) == 0 and q(112, 32, 3) == 0 and q(0, 32, 1) == 0

    def fused(cin):
        sdfg = graphs.mbconv_block(1, cin, 32, expand=2, cout=24, se_reduce=4, stride=2, dtype=torch.float32)
        return fusion.auto_optimize(sdfg)["expand_depthwise"]
    assert fused(1024) == 1      # 13 KB of rows + 131 KB of weights: fits
    assert fused(1200) == 0      # 154 KB of weights alone: the launch would be refused
