"""Node forms outside the measured configurations: Reduce* over axes that are not adjacent
(pure_implementations.py:101-103,294-306 take any ``axes``) and the Softmax reverse node for an axis other than the
last (DefaultSoftmaxBackward, daceml/autodiff/implementations/onnx_ops.py:237-275, reduces over the single axis
``axis``). Both are compositions of kernels that exist: several reduction passes, and the reference's own Mul /
ReduceSum / Mul / Sub.

As in test_zy_gemm_node.py each case runs twice: on a GPU through the kernels, and without a GPU with the emitted
calls interpreted by tests/abi_emulator.py (which checks the lowering, not the kernels)."""
import numpy as np
import pytest
import torch

from oracle import ops as O
from tests.util import assert_close, dev, first_run_on_hardware, host, rng

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


@first_run_on_hardware("written without access to a GPU: first run on hardware")
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
    want = O.softmax_backward(y.astype(np.float64), dy.astype(np.float64), axis % len(shape))
    tol = dict(rtol=2e-2, atol=1e-2) if dtype == torch.float16 else dict(rtol=1e-5, atol=1e-6)
    assert_close(arrays["gradient_x"], want, dtype, "emulated softmax backward %s axis %d" % (shape, axis), **tol)


@first_run_on_hardware("written without access to a GPU: first run on hardware")
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
    want = O.softmax_backward(host(y).astype(np.float64), dy.astype(np.float64), axis % len(shape))
    assert_close(host(dx), want, dtype, "softmax backward %s axis %d" % (shape, axis), **tol)
