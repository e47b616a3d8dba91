"""ONNXGemm (PureGemm, daceml/onnx/op_implementations/pure_implementations.py:380-553) with every attribute:
transA / transB, alpha, beta in {0, 1, other}, C as a vector over the last result index, as ``[1, N]`` and as a full
``[M, N]`` matrix - against ``oracle.ops.gemm``.

Two runs of the same cases: on a GPU through the library-node path and the kernels; and, without a GPU, the calls the
expansion emits interpreted by ``tests/abi_emulator.py`` (checks the lowering: descriptors, operand order, workspace
layout, the extra scaling launch)."""
import itertools

import numpy as np
import pytest
import torch

from oracle import ops as O
from tests.util import assert_close, dev, host, rng

M, N, K = 24, 40, 64

#: (transA, transB, alpha, beta, kind of C)
CASES = [(ta, tb, alpha, beta, ckind)
         for (ta, tb), (alpha, beta, ckind) in itertools.product(
             [(0, 0), (0, 1), (1, 0), (1, 1)],
             [(1.0, 0.0, None), (1.0, 1.0, "n"), (0.5, 1.0, "n"), (1.0, 1.0, "mn"), (0.25, 0.5, "n"), (2.0, 0.5, "mn"),
              (1.0, -1.5, "1n"), (1.0, 1.0, "1n"), (1.5, 0.0, "n")])]


def _case(dtype, ta, tb, alpha, beta, ckind, seed=5):
    """The node on an SDFG of its own plus seeded operands (rounded to `dtype`) and the oracle's result."""
    from daceml_amd import graphs
    npdt = np.float16 if dtype == torch.float16 else np.float32
    r = rng(seed)
    a = (r.standard_normal((K, M) if ta else (M, K)) * 0.5).astype(npdt)
    b = (r.standard_normal((N, K) if tb else (K, N)) * 0.5).astype(npdt)
    c = None
    if ckind is not None:
        c = r.standard_normal({"n": (N, ), "1n": (1, N), "mn": (M, N)}[ckind]).astype(npdt)
    g = graphs.GraphBuilder("gemm", dtype)
    ins = {"A": g.input("a", a.shape), "B": g.input("b", b.shape)}
    if c is not None:
        ins["C"] = g.input("c", c.shape)
    y = g.node("Gemm", ins, {"Y": (M, N)}, label="gemm", alpha=alpha, beta=beta, transA=ta, transB=tb)["Y"]
    g.output(y, "y")
    c64 = None if c is None else c.astype(np.float64).reshape(-1) if ckind == "1n" else c.astype(np.float64)
    want = O.gemm(a.astype(np.float64), b.astype(np.float64), c64, alpha=alpha, beta=beta, transA=ta, transB=tb)
    return g, a, b, c, want


def _tolerance(dtype):
    # K = 64 products of N(0, 0.25) values: the un-widened bounds hold
    return dict(rtol=2e-2, atol=1e-2) if dtype == torch.float16 else dict(rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
@pytest.mark.parametrize("ta,tb,alpha,beta,ckind", CASES)
def test_gemm_expansion_asks_for_the_right_calls(dtype, ta, tb, alpha, beta, ckind):
    from tests.abi_emulator import Emulator
    g, a, b, c, want = _case(dtype, ta, tb, alpha, beta, ckind)
    node = g.state.library_nodes()[0]
    tasklet = node.expand(g.sdfg, g.state)
    scaled = ckind is not None and beta not in (0.0, 1.0)
    assert [call.symbol.rsplit("_", 1)[0] if "unary" in call.symbol else "gemm" for call in tasklet.calls] == \
        (["dmlhip_unary", "gemm"] if scaled else ["gemm"])
    y = np.full((M, N), np.nan, dtype=a.dtype)
    arrays = {"A": a.copy(), "B": b.copy(), "Y": y}
    if c is not None:
        arrays["C"] = c.copy()
    em = Emulator(tasklet.workspace_bytes)
    em.run(tasklet, arrays)
    assert_close(y, want, dtype, "emulated Gemm %s" % ((ta, tb, alpha, beta, ckind), ), **_tolerance(dtype))
    # inputs are untouched (the scaled C goes to the workspace or to Y, never back into C)
    assert np.array_equal(arrays["A"], a) and np.array_equal(arrays["B"], b)
    if c is not None:
        assert np.array_equal(arrays["C"], c)
    if scaled and ckind != "mn":
        assert tasklet.workspace_bytes >= 256, "the scaled vector lives in the workspace"


def test_gemm_refuses_what_the_reference_refuses():
    """C must broadcast by the reference's rule (trailing dims equal, :533-539): a column vector [M, 1] or a scalar
    does not; 1-D operands are not Gemm operands."""
    from daceml_amd import graphs
    import daceml_amd.onnx as donnx
    for c_shape in ((M, 1), (1, ), (N + 1, )):
        g = graphs.GraphBuilder("gemm", torch.float32)
        ins = {"A": g.input("a", (M, K)), "B": g.input("b", (K, N)), "C": g.input("c", c_shape)}
        g.output(g.node("Gemm", ins, {"Y": (M, N)}, label="gemm")["Y"], "y")
        node = g.state.library_nodes()[0]
        with pytest.raises(donnx.NotApplicable):
            node.expand(g.sdfg, g.state)
    with pytest.raises(ValueError):
        O.gemm(np.zeros((M, K)), np.zeros((K, N)), np.zeros((M, 1)))


def _gemm_gradients(a, b, c, dy, ta, tb, alpha, beta, ckind):
    """Autograd in fp64 on the definition Y = alpha op(A) op(B) + beta C."""
    ta_, tb_ = (torch.tensor(t.astype(np.float64), requires_grad=True) for t in (a, b))
    tc = None if c is None else torch.tensor(c.astype(np.float64), requires_grad=True)
    y = alpha * ((ta_.T if ta else ta_) @ (tb_.T if tb else tb_))
    if tc is not None:
        y = y + beta * tc
    y.backward(torch.tensor(dy.astype(np.float64)))
    return ta_.grad.numpy(), tb_.grad.numpy(), None if tc is None or beta == 0 else tc.grad.numpy()


BACKWARD_CASES = [c for c in CASES if c[:2] in ((0, 0), (1, 1), (0, 1))]


def _backward_graph(dtype, ta, tb, alpha, beta, ckind):
    from daceml_amd.autodiff import add_backward_pass
    g, a, b, c, want = _case(dtype, ta, tb, alpha, beta, ckind)
    wrt = ["a", "b"] + (["c"] if c is not None and beta != 0 else [])
    grads = add_backward_pass(g.sdfg, g.state, ["y"], wrt)
    assert grads == {n: "gradient_" + n for n in wrt}
    dy = rng(9).standard_normal((M, N)).astype(a.dtype)
    return g, a, b, c, dy, wrt


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
@pytest.mark.parametrize("ta,tb,alpha,beta,ckind", BACKWARD_CASES)
def test_gemm_reverse_node_lowers_correctly(dtype, ta, tb, alpha, beta, ckind):
    """Gemm has a reverse implementation of its own (A and B as for the Einsum PureGemm builds, C = beta times the
    incoming gradient, summed over the rows for a vector): checked against autograd through the emulated calls."""
    from daceml_amd.runtime import expand_onnx_nodes
    from tests.abi_emulator import run_sdfg
    g, a, b, c, dy, wrt = _backward_graph(dtype, ta, tb, alpha, beta, ckind)
    expand_onnx_nodes(g.sdfg)
    arrays = {"a": a.copy(), "b": b.copy(), "gradient_y": dy.copy()}
    if c is not None:
        arrays["c"] = c.copy()
    run_sdfg(g.sdfg, arrays)
    wa, wb, wc = _gemm_gradients(a, b, c, dy, ta, tb, alpha, beta, ckind)
    tol = dict(rtol=2e-2, atol=2e-2) if dtype == torch.float16 else dict(rtol=1e-5, atol=2e-6)
    assert_close(arrays["gradient_a"], wa, dtype, "dA %s" % ((ta, tb, alpha, beta, ckind), ), **tol)
    assert_close(arrays["gradient_b"], wb, dtype, "dB", **tol)
    if "c" in wrt:
        assert arrays["gradient_c"].shape == c.shape
        assert_close(arrays["gradient_c"], wc, dtype, "dC", **(tol if dtype == torch.float32 else dict(rtol=2e-2, atol=5e-2)))


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
@pytest.mark.parametrize("ta,tb,alpha,beta,ckind", BACKWARD_CASES[::3])
def test_gemm_backward_on_gpu(dtype, ta, tb, alpha, beta, ckind):
    from daceml_amd.runtime import CompiledSDFG
    g, a, b, c, dy, wrt = _backward_graph(dtype, ta, tb, alpha, beta, ckind)
    prog = CompiledSDFG(g.sdfg)
    args = {"a": dev(a), "b": dev(b), "y": torch.empty((M, N), dtype=dtype, device="cuda"), "gradient_y": dev(dy)}
    if c is not None:
        args["c"] = dev(c)
    outs = {n: torch.full(tuple(g.sdfg.arrays["gradient_" + n].shape), float("nan"), dtype=dtype, device="cuda") for n in wrt}
    prog(**args, **{"gradient_" + n: t for n, t in outs.items()})
    wa, wb, wc = _gemm_gradients(a, b, c, dy, ta, tb, alpha, beta, ckind)
    tol = dict(rtol=2e-2, atol=2e-2) if dtype == torch.float16 else dict(rtol=1e-5, atol=2e-6)
    assert_close(host(outs["a"]), wa, dtype, "dA %s" % ((ta, tb, alpha, beta, ckind), ), **tol)
    assert_close(host(outs["b"]), wb, dtype, "dB", **tol)
    if "c" in wrt:
        assert_close(host(outs["c"]), wc, dtype, "dC", **(tol if dtype == torch.float32 else dict(rtol=2e-2, atol=5e-2)))


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
@pytest.mark.parametrize("ta,tb,alpha,beta,ckind", CASES)
def test_gemm_node_on_gpu(dtype, ta, tb, alpha, beta, ckind):
    from daceml_amd.runtime import CompiledSDFG
    g, a, b, c, want = _case(dtype, ta, tb, alpha, beta, ckind)
    prog = CompiledSDFG(g.sdfg)
    y = torch.full((M, N), float("nan"), dtype=dtype, device="cuda")
    args = {"a": dev(a), "b": dev(b), "y": y}
    if c is not None:
        args["c"] = dev(c)
    prog(**args)
    assert_close(host(y), want, dtype, "Gemm %s" % ((ta, tb, alpha, beta, ckind), ), **_tolerance(dtype))
    if c is not None:
        assert np.array_equal(host(args["c"]), c.astype(np.float32) if dtype == torch.float16 else c)


class AddMM(torch.nn.Module):
    """nn.Linear on a 2-D input exports to Gemm(transB=1) with the bias as C; ``torch.addmm`` with scalars exports to
    Gemm with alpha, beta and a full matrix C."""
    def __init__(self):
        super().__init__()
        self.fc = torch.nn.Linear(K, N)

    def forward(self, bias, x, w):
        return torch.addmm(bias, self.fc(x), w, beta=0.5, alpha=2.0)


def test_exported_gemm_nodes_keep_their_attributes_and_lower_correctly():
    """The exporter's Gemm nodes, imported and expanded, then interpreted on the CPU: the node sequence, attributes
    and the numerical result of the emitted calls match the eager module."""
    from daceml_amd.runtime import expand_onnx_nodes
    from daceml_amd.torch import DaceModule
    from tests.abi_emulator import run_state
    torch.manual_seed(3)
    net = AddMM()
    bias, x, w = torch.randn(M, N), torch.randn(M, K) * 0.5, torch.randn(N, N) * 0.2
    model = DaceModule(net)._import((bias, x, w))
    st = model.sdfg.states()[0]
    gemm = [n for n in st.library_nodes() if n.schema.name == "Gemm"]
    assert len(gemm) == 1 and (gemm[0].alpha, gemm[0].beta, gemm[0].transA, gemm[0].transB) == (2.0, 0.5, 0, 0)
    expand_onnx_nodes(model.sdfg)
    from daceml_amd.onnx.onnx_importer import clean_onnx_name
    names = [clean_onnx_name(n) for n in model.inputs]
    arrays = dict(zip(names, [t.numpy().copy() for t in (bias, x, w)] +
                      [net.fc.weight.detach().numpy().copy(), net.fc.bias.detach().numpy().copy()]))
    em = run_state(model.sdfg, st, arrays)
    assert em.log == ["dmlhip_gemm_f32", "dmlhip_unary_f32", "dmlhip_gemm_f32"]
    want = net.double()(bias.double(), x.double(), w.double()).detach().numpy()
    assert_close(arrays[model.outputs[0]], want, torch.float32, "addmm through Gemm nodes (emulated)", rtol=1e-5, atol=2e-6)


@pytest.mark.gpu
def test_gemm_node_through_the_module_wrapper():
    from daceml_amd.torch import DaceModule
    torch.manual_seed(3)
    net = AddMM().cuda()
    bias = torch.randn(M, N, device="cuda")
    x = torch.randn(M, K, device="cuda") * 0.5
    w = torch.randn(N, N, device="cuda") * 0.2
    wrapped = DaceModule(net)
    got = wrapped(bias, x, w)
    want = net.double()(bias.double(), x.double(), w.double())
    kinds = [n.kind for n in wrapped.compiled.sdfg.states()[0].library_nodes()]
    assert kinds.count("gemm") >= 2
    assert_close(host(got), want.detach().cpu().numpy(), torch.float32, "addmm through Gemm nodes", rtol=1e-5, atol=2e-6)
