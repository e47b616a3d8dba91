"""Node forms outside the measured configurations: Reduce* over axes that are not adjacent
(pure_implementations.py:101-103,294-306 take any ``axes``) and the Softmax reverse node for an axis other than the
last (DefaultSoftmaxBackward, daceml/autodiff/implementations/onnx_ops.py:237-275; summed over every axis the forward
made one row of, see oracle.ops.softmax_backward_rows). Both are compositions of kernels that exist: several reduction passes, and the reference's own Mul /
ReduceSum / Mul / Sub.

As in test_zy_gemm_node.py each case runs twice: on a GPU through the kernels, and without a GPU with the emitted
calls interpreted by tests/abi_emulator.py (which checks the lowering, not the kernels)."""
import numpy as np
import pytest
import torch

from oracle import ops as O
from tests.util import assert_close, dev, host, rng

REDUCE_CASES = [((4, 6, 8), [0, 2]), ((3, 5, 7, 9), [0, 2]), ((3, 5, 7, 9), [1, 3]), ((2, 3, 4, 5, 6), [0, 2, 4]),
                ((6, 1, 5, 4), [0, 3]), ((4, 6, 8), [0, 1])]


def _reduce_graph(dtype, name, shape, axes, keepdims):
    from daceml_amd import graphs
    g = graphs.GraphBuilder("reduce", dtype)
    x = g.input("x", shape)
    want_shape = O.reduce_sum(np.zeros(shape), axes, keepdims).shape
    y = g.node("Reduce" + name.capitalize(), {"data": x}, {"reduced": want_shape}, label="red", axes=list(axes),
               keepdims=keepdims)["reduced"]
    g.output(y, "y")
    return g, want_shape


def _reduce_data(dtype, name, shape, axes, keepdims):
    npdt = np.float16 if dtype == torch.float16 else np.float32
    x = rng(41).standard_normal(shape).astype(npdt)
    want = getattr(O, "reduce_" + name)(x.astype(np.float64), axes, keepdims)
    n = x.size // max(want.size, 1)
    if dtype == torch.float16:
        tol = dict(rtol=2e-2, atol=1e-2)
    else:
        tol = dict(rtol=1e-5, atol=1e-6 * max(1.0, np.sqrt(n)) if name == "sum" else 1e-6)
    return x, want, tol


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
@pytest.mark.parametrize("name", ["sum", "mean", "max", "min"])
@pytest.mark.parametrize("shape,axes", REDUCE_CASES)
@pytest.mark.parametrize("keepdims", [1, 0])
def test_reduce_over_separate_axes_lowers_to_passes(dtype, name, shape, axes, keepdims):
    from tests.abi_emulator import run_state
    from daceml_amd.runtime import expand_onnx_nodes
    g, want_shape = _reduce_graph(dtype, name, shape, axes, keepdims)
    x, want, tol = _reduce_data(dtype, name, shape, axes, keepdims)
    expand_onnx_nodes(g.sdfg)
    arrays = {"x": x.copy()}
    em = run_state(g.sdfg, g.state, arrays)
    runs = 1 + sum(1 for a, b in zip(sorted(axes), sorted(axes)[1:]) if b != a + 1)
    assert len(em.log) == runs and all(s.startswith("dmlhip_reduce_") for s in em.log)
    assert em.log[0].endswith("f16" if dtype == torch.float16 else "f32") and all(s.endswith("f32") for s in em.log[1:])
    assert arrays["y"].shape == want.shape
    assert_close(arrays["y"], want, dtype, "emulated reduce_%s %s %s" % (name, shape, axes), **tol)
    assert np.array_equal(arrays["x"], x)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
@pytest.mark.parametrize("name", ["sum", "mean", "max", "min"])
@pytest.mark.parametrize("shape,axes", REDUCE_CASES)
@pytest.mark.parametrize("keepdims", [1, 0])
def test_reduce_over_separate_axes_on_gpu(dtype, name, shape, axes, keepdims):
    from daceml_amd.runtime import CompiledSDFG
    g, want_shape = _reduce_graph(dtype, name, shape, axes, keepdims)
    x, want, tol = _reduce_data(dtype, name, shape, axes, keepdims)
    prog = CompiledSDFG(g.sdfg)
    y = torch.full(want_shape, float("nan"), dtype=dtype, device="cuda")
    prog(x=dev(x), y=y)
    assert_close(host(y), want, dtype, "reduce_%s %s %s" % (name, shape, axes), **tol)


SOFTMAX_CASES = [((4, 6, 16), 1), ((3, 5, 7, 9), 2), ((3, 5, 7, 9), 0), ((4, 6, 16), -1), ((5, 33), 0)]


def _softmax_backward_graph(dtype, shape, axis):
    from daceml_amd import graphs
    from daceml_amd.autodiff import add_backward_pass
    g = graphs.GraphBuilder("softmax", dtype)
    x = g.input("x", shape)
    g.output(g.node("Softmax", {"input": x}, {"output": shape}, label="sm", axis=axis)["output"], "y")
    grads = add_backward_pass(g.sdfg, g.state, ["y"], ["x"])
    assert grads == {"x": "gradient_x"}
    return g


def _softmax_backward_data(dtype, shape, axis):
    npdt = np.float16 if dtype == torch.float16 else np.float32
    r = rng(43)
    x = r.standard_normal(shape).astype(npdt)
    dy = r.standard_normal(shape).astype(npdt)
    y64 = O.softmax(x.astype(np.float64), axis=axis)
    return x, dy, y64


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
@pytest.mark.parametrize("shape,axis", SOFTMAX_CASES)
def test_softmax_reverse_node_for_any_axis_lowers_correctly(dtype, shape, axis):
    """The backward state alone, fed with the forward output as the oracle computes it."""
    from tests.abi_emulator import run_state
    from daceml_amd.runtime import expand_onnx_nodes
    g = _softmax_backward_graph(dtype, shape, axis)
    bst = g.sdfg.states()[1]
    names = sorted(n.schema.name for n in bst.library_nodes())
    last = axis % len(shape) == len(shape) - 1
    assert names == (["SoftmaxGrad"] if last else ["Mul", "Mul", "ReduceSum", "Sub"])
    x, dy, y64 = _softmax_backward_data(dtype, shape, axis)
    y = y64.astype(x.dtype)
    expand_onnx_nodes(g.sdfg)
    arrays = {"y": y.copy(), "gradient_y": dy.copy()}
    run_state(g.sdfg, bst, arrays)
    want = O.softmax_backward_rows(y.astype(np.float64), dy.astype(np.float64), axis % len(shape))
    tol = dict(rtol=2e-2, atol=1e-2) if dtype == torch.float16 else dict(rtol=1e-5, atol=1e-6)
    assert_close(arrays["gradient_x"], want, dtype, "emulated softmax backward %s axis %d" % (shape, axis), **tol)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
@pytest.mark.parametrize("shape,axis", SOFTMAX_CASES)
def test_softmax_backward_for_any_axis_on_gpu(dtype, shape, axis):
    from daceml_amd.runtime import CompiledSDFG
    g = _softmax_backward_graph(dtype, shape, axis)
    x, dy, y64 = _softmax_backward_data(dtype, shape, axis)
    prog = CompiledSDFG(g.sdfg)
    y = torch.empty(shape, dtype=dtype, device="cuda")
    dx = torch.full(shape, float("nan"), dtype=dtype, device="cuda")
    prog(x=dev(x), y=y, gradient_y=dev(dy), gradient_x=dx)
    tol = dict(rtol=2e-2, atol=1e-2) if dtype == torch.float16 else dict(rtol=1e-5, atol=1e-6)
    assert_close(host(y), y64, dtype, "softmax %s axis %d" % (shape, axis), **tol)
    # the reverse node reads the forward output as the kernel rounded it
    want = O.softmax_backward_rows(host(y).astype(np.float64), dy.astype(np.float64), axis % len(shape))
    assert_close(host(dx), want, dtype, "softmax backward %s axis %d" % (shape, axis), **tol)


# ----------------------------------------------------------------------------- LogSoftmax
LOG_SOFTMAX_CASES = [((8, 10), 1), ((3, 4, 33), -1), ((2, 3, 4, 5), 1), ((6, 40), 0), ((2, 300), 1)]


def _log_softmax_graph(dtype, shape, axis, backward):
    from daceml_amd import graphs
    from daceml_amd.autodiff import add_backward_pass
    g = graphs.GraphBuilder("log_softmax", dtype)
    y = g.node("LogSoftmax", {"input": g.input("x", shape)}, {"output": shape}, label="lsm", axis=axis)["output"]
    g.output(y, "y")
    if backward:
        add_backward_pass(g.sdfg, g.state, ["y"], ["x"])
    return g


def _log_softmax_data(dtype, shape):
    npdt = np.float16 if dtype == torch.float16 else np.float32
    r = rng(47)
    x = (r.standard_normal(shape) * 4).astype(npdt)
    x.reshape(-1)[::7] -= 30          # probabilities that fp16 cannot hold: their logarithms still have to come out
    return x, r.standard_normal(shape).astype(npdt)


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
@pytest.mark.parametrize("shape,axis", LOG_SOFTMAX_CASES)
def test_log_softmax_lowers_to_the_reference_statements(dtype, shape, axis):
    """Six calls in the pure expansion's order (pure_implementations.py:649-656); the reverse is the reference's
    Exp / ReduceSum / Mul / Sub (onnx_ops.py:338-373) over all the axes of a row."""
    from tests.abi_emulator import run_sdfg
    from daceml_amd.runtime import expand_onnx_nodes
    g = _log_softmax_graph(dtype, shape, axis, backward=True)
    assert sorted(n.schema.name for n in g.sdfg.states()[1].library_nodes()) == ["Exp", "Mul", "ReduceSum", "Sub"]
    expand_onnx_nodes(g.sdfg)
    x, dy = _log_softmax_data(dtype, shape)
    arrays = {"x": x.copy(), "gradient_y": dy.copy()}
    log = run_sdfg(g.sdfg, arrays)
    sfx = "f16" if dtype == torch.float16 else "f32"
    assert log[:6] == ["dmlhip_%s_%s" % (k, sfx) for k in ("reduce", "binary", "unary", "reduce", "unary", "binary")]
    ax = axis % len(shape)
    want = O.log_softmax(x.astype(np.float64), ax)
    assert np.isfinite(arrays["y"]).all()
    tol = dict(rtol=2e-2, atol=2e-2) if dtype == torch.float16 else dict(rtol=1e-5, atol=2e-6)
    assert_close(arrays["y"], want, dtype, "emulated LogSoftmax %s axis %d" % (shape, axis), **tol)
    # the reverse reads the forward output as the kernels rounded it; the sum runs over the whole row
    y = arrays["y"].astype(np.float64)
    dy64 = dy.astype(np.float64)
    want_dx = dy64 - np.exp(y) * dy64.sum(axis=tuple(range(ax, len(shape))), keepdims=True)
    assert_close(arrays["gradient_x"], want_dx, dtype, "emulated LogSoftmax reverse %s axis %d" % (shape, axis),
                 **(dict(rtol=2e-2, atol=3e-2) if dtype == torch.float16 else dict(rtol=1e-5, atol=1e-5)))
    if ax == len(shape) - 1:
        np.testing.assert_allclose(want_dx, O.log_softmax_backward(y, dy64, ax), rtol=1e-12, atol=1e-12)


def test_exported_log_softmax_head():
    """A classifier head as LeNet ends (tests/torch/test_lenet.py of the reference): Linear, LogSoftmax."""
    from daceml_amd.onnx.onnx_importer import clean_onnx_name
    from daceml_amd.runtime import expand_onnx_nodes
    from daceml_amd.torch import DaceModule
    from tests.abi_emulator import run_state

    class Head(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.fc = torch.nn.Linear(84, 10)

        def forward(self, x):
            return torch.nn.functional.log_softmax(self.fc(x), dim=1)

    torch.manual_seed(8)
    net, x = Head(), torch.randn(8, 84)
    model = DaceModule(net)._import((x, ))
    st = model.sdfg.states()[0]
    assert "LogSoftmax" in [n.schema.name for n in st.library_nodes()]
    expand_onnx_nodes(model.sdfg)
    names = [clean_onnx_name(n) for n in model.inputs]
    arrays = dict(zip(names, [x.numpy().copy()] + [p.detach().numpy().copy() for p in net.parameters()]))
    run_state(model.sdfg, st, arrays)
    assert_close(arrays[model.outputs[0]], net.double()(x.double()).detach().numpy(), torch.float32, "Linear + LogSoftmax",
                 rtol=1e-5, atol=2e-6)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
@pytest.mark.parametrize("shape,axis", LOG_SOFTMAX_CASES)
def test_log_softmax_on_gpu(dtype, shape, axis):
    from daceml_amd.runtime import CompiledSDFG
    g = _log_softmax_graph(dtype, shape, axis, backward=True)
    x, dy = _log_softmax_data(dtype, shape)
    prog = CompiledSDFG(g.sdfg)
    y = torch.full(shape, float("nan"), dtype=dtype, device="cuda")
    dx = torch.full(shape, float("nan"), dtype=dtype, device="cuda")
    prog(x=dev(x), y=y, gradient_y=dev(dy), gradient_x=dx)
    ax = axis % len(shape)
    tol = dict(rtol=2e-2, atol=2e-2) if dtype == torch.float16 else dict(rtol=1e-5, atol=2e-6)
    assert_close(host(y), O.log_softmax(x.astype(np.float64), ax), dtype, "LogSoftmax %s axis %d" % (shape, axis), **tol)
    y64, dy64 = host(y).astype(np.float64), dy.astype(np.float64)
    want_dx = dy64 - np.exp(y64) * dy64.sum(axis=tuple(range(ax, len(shape))), keepdims=True)
    assert_close(host(dx), want_dx, dtype, "LogSoftmax reverse %s axis %d" % (shape, axis),
                 **(dict(rtol=2e-2, atol=3e-2) if dtype == torch.float16 else dict(rtol=1e-5, atol=1e-5)))
