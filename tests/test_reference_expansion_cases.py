"""The cases of the reference's expansion tests (tests/pure_expansions/test_expansions.py) that lie on this path - MatMul
[2,4] x [4,3] (:21-62), the nine Reduce cases over a [2,4,10] tensor (:186-238), Reshape to [8,10] / [80] / [2,40]
(:281-317), Reciprocal (:353-384), Einsum ``bij,jk->bik`` (:387-406), Reshape followed by a broadcast Add (:409-429), Sum
of three arrays (:432-461) - as single-node graphs whose expansions' calls are interpreted on the CPU
(tests/abi_emulator.py) and compared with NumPy as the reference's tests do. fp32 throughout (the reference's Einsum and
reshape-add cases are fp64, which this path does not compute in)."""
import numpy as np
import pytest
import torch


def _run(g, arrays):
    from daceml_amd.runtime import expand_onnx_nodes
    from tests.abi_emulator import run_state
    expand_onnx_nodes(g.sdfg)
    run_state(g.sdfg, g.state, arrays)
    return arrays["y"]


def _builder(name):
    from daceml_amd import graphs
    return graphs.GraphBuilder(name, torch.float32)


def test_matmul_expansion():
    r = np.random.default_rng(0)
    x, z = r.random((2, 4), dtype=np.float32), r.random((4, 3), dtype=np.float32)
    g = _builder("matmul")
    g.output(g.node("MatMul", {"A": g.input("x", (2, 4)), "B": g.input("z", (4, 3))}, {"Y": (2, 3)}, label="Matmul")["Y"], "y")
    np.testing.assert_allclose(_run(g, {"x": x, "z": z}), x @ z, rtol=1e-6)


@pytest.mark.parametrize("reduce_type,keepdims,axes", [("Sum", True, [0]), ("Sum", False, [-1]), ("Sum", True, [0, -1]),
                                                        ("Max", False, [0, -1]), ("Max", True, [0]), ("Max", True, [-1]),
                                                        ("Mean", True, [-1]), ("Mean", True, [0, -1]), ("Mean", False, [0])])
def test_reduce(reduce_type, keepdims, axes):
    x = np.random.default_rng(1).normal(scale=10, size=(2, 4, 10)).astype(np.float32)
    want = getattr(np, reduce_type.lower())(x.copy(), axis=tuple(axes), keepdims=keepdims)
    g = _builder("reduce")
    g.output(g.node("Reduce" + reduce_type, {"data": g.input("x", (2, 4, 10))}, {"reduced": want.shape}, label="reduce",
                    axes=axes, keepdims=1 if keepdims else 0)["reduced"], "y")
    np.testing.assert_allclose(_run(g, {"x": x}), want, rtol=1e-5, atol=1e-5)


def test_reduce_to_a_scalar():
    """test_reduce_scalar (:241-278) / the ONNX scalar-return regression: a 1-D ReduceSum without keepdims."""
    x = np.arange(5, dtype=np.float32)
    g = _builder("reduce_scalar")
    g.output(g.node("ReduceSum", {"data": g.input("x", (5, ))}, {"reduced": ()}, label="reduce", keepdims=0)["reduced"], "y")
    out = _run(g, {"x": x})
    assert out.shape == () and out[()] == 1 + 2 + 3 + 4


@pytest.mark.parametrize("new_shape", [[8, 10], [80], [2, 40]])
def test_reshape(new_shape):
    x = np.random.default_rng(2).normal(scale=10, size=(2, 4, 10)).astype(np.float32)
    g = _builder("reshape")
    g.output(g.node("Reshape", {"data": g.input("x", (2, 4, 10))}, {"reshaped": tuple(new_shape)}, label="reshape")["reshaped"],
             "y")
    np.testing.assert_array_equal(_run(g, {"x": x}), x.reshape(*new_shape))


def test_reciprocal():
    x = np.random.default_rng(3).normal(scale=10, size=(2, 4, 10)).astype(np.float32)
    g = _builder("reciprocal")
    g.output(g.node("Reciprocal", {"X": g.input("x", (2, 4, 10))}, {"Y": (2, 4, 10)}, label="reciprocal")["Y"], "y")
    np.testing.assert_allclose(_run(g, {"x": x}), 1 / x, rtol=1e-6)


def test_einsum():
    r = np.random.default_rng(4)
    a, b = r.random((5, 4, 3), dtype=np.float32), r.random((3, 2), dtype=np.float32)
    g = _builder("einsum")
    g.output(g.node("Einsum", {"Inputs__0": g.input("a", (5, 4, 3)), "Inputs__1": g.input("b", (3, 2))}, {"Output": (5, 4, 2)},
                    label="einsum", equation="bij, jk -> bik")["Output"], "y")
    np.testing.assert_allclose(_run(g, {"a": a, "b": b}), np.einsum("bij ,jk -> bik", a, b), rtol=1e-6)


def test_reshape_add():
    inp, bias = np.arange(9).astype(np.float32), np.arange(3).astype(np.float32)
    g = _builder("reshape_add")
    reshaped = g.node("Reshape", {"data": g.input("inp", (9, ))}, {"reshaped": (3, 3)}, label="reshape")["reshaped"]
    g.output(g.node("Add", {"A": reshaped, "B": g.input("bias", (3, ))}, {"C": (3, 3)}, label="add")["C"], "y")
    np.testing.assert_array_equal(_run(g, {"inp": inp, "bias": bias}), inp.reshape(3, 3) + bias)


@pytest.mark.parametrize("shape", [(2, 3), (1, )])
def test_sum_arrays(shape):
    r = np.random.default_rng(5)
    inputs = [r.standard_normal(shape).astype(np.float32) for _ in range(3)]
    g = _builder("sum_arrays")
    ins = {"data_0__%d" % i: g.input("inp%d" % i, shape) for i in range(3)}
    g.output(g.node("Sum", ins, {"sum": shape}, label="sum")["sum"], "y")
    np.testing.assert_allclose(_run(g, {"inp%d" % i: v for i, v in enumerate(inputs)}), (inputs[0] + inputs[1]) + inputs[2],
                               rtol=1e-6)
