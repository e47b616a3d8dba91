"""1-D Conv nodes (CudnnConvolution takes them as [N, C, L, 1], cudnn_implementations.py:20-66,243-250): here they are
lowered to the 2-D kernels as [N, C, 1, L] with a 1 x k filter. Oracle: ``oracle.ops.conv2d`` on the same reshaping,
itself checked here against ``torch.nn.functional.conv1d``.

The host-side tests interpret the emitted calls with tests/abi_emulator.py; the GPU tests run small problems (direct
kernel and contraction kernels) and one long sequence that is large enough for the implicit-GEMM kernel, which then
runs with a single output row."""
import numpy as np
import pytest
import torch

from oracle import ops as O
from tests.util import assert_close, dev, host, rng

# n, c, l, m, k, stride, pad, dilation, group, bias
CASES = [(2, 3, 40, 8, 3, 1, 1, 1, 1, True), (3, 4, 33, 6, 5, 2, 2, 1, 2, False), (1, 8, 100, 8, 3, 1, 2, 2, 8, True),
         (2, 16, 64, 32, 1, 1, 0, 1, 1, True), (2, 5, 7, 4, 7, 1, 0, 1, 1, False), (1, 2, 130, 3, 4, 3, 1, 1, 1, True)]


def _data(n, c, l, m, k, stride, pad, dil, group, bias, dtype=np.float32):
    r = rng(61)
    x = r.standard_normal((n, c, l)).astype(dtype)
    w = (r.standard_normal((m, c // group, k)) / np.sqrt(c // group * k)).astype(dtype)
    b = r.standard_normal(m).astype(dtype) if bias else None
    want = O.conv2d(x.astype(np.float64)[:, :, None, :], w.astype(np.float64)[:, :, None, :],
                    None if b is None else b.astype(np.float64), (1, stride), (0, pad, 0, pad), (1, dil), group)[:, :, 0, :]
    return x, w, b, want


def _graph(dtype, n, c, l, m, k, stride, pad, dil, group, bias, out_l):
    from daceml_amd import graphs
    g = graphs.GraphBuilder("conv1d", dtype)
    ins = {"X": g.input("x", (n, c, l)), "W": g.input("w", (m, c // group, k))}
    if bias:
        ins["B"] = g.input("b", (m, ))
    y = g.node("Conv", ins, {"Y": (n, m, out_l)}, label="conv", kernel_shape=[k], strides=[stride], pads=[pad, pad],
               dilations=[dil], group=group)["Y"]
    g.output(y, "y")
    return g


@pytest.mark.parametrize("case", CASES)
def test_the_oracle_on_the_reshaped_problem_is_conv1d(case):
    n, c, l, m, k, stride, pad, dil, group, bias = case
    x, w, b, want = _data(*case, dtype=np.float64)
    ref = torch.nn.functional.conv1d(torch.tensor(x), torch.tensor(w), None if b is None else torch.tensor(b), stride=stride,
                                     padding=pad, dilation=dil, groups=group)
    np.testing.assert_allclose(want, ref.numpy(), rtol=1e-12, atol=1e-12)


@pytest.mark.parametrize("case", CASES)
def test_conv1d_lowers_to_one_2d_call(case):
    from daceml_amd.runtime import expand_onnx_nodes
    from tests.abi_emulator import run_state
    n, c, l, m, k, stride, pad, dil, group, bias = case
    x, w, b, want = _data(*case)
    g = _graph(torch.float32, *case, out_l=want.shape[2])
    expand_onnx_nodes(g.sdfg)
    arrays = {"x": x.copy(), "w": w.copy()}
    if bias:
        arrays["b"] = b.copy()
    em = run_state(g.sdfg, g.state, arrays)
    assert em.log == ["dmlhip_conv2d_f32"]
    desc = [a for a in g.state.library_nodes()[0].calls[0].args if hasattr(a, "value") and hasattr(a.value, "kh")][0].value
    assert (desc.h, desc.w, desc.kh, desc.kw) == (1, l, 1, k)
    assert (desc.stride_h, desc.stride_w, desc.pad_h, desc.pad_w, desc.dil_h, desc.dil_w) == (1, stride, 0, pad, 1, dil)
    assert arrays["y"].shape == want.shape
    assert_close(arrays["y"], want, torch.float32, "emulated conv1d %s" % (case, ), rtol=1e-5, atol=2e-6)


def test_conv1d_backward_lowers_to_the_2d_gradient_calls():
    from daceml_amd.autodiff import add_backward_pass
    from daceml_amd.runtime import expand_onnx_nodes
    from tests.abi_emulator import run_state
    case = CASES[1]
    n, c, l, m, k, stride, pad, dil, group, bias = case
    x, w, b, want = _data(*case)
    g = _graph(torch.float32, *case, out_l=want.shape[2])
    grads = add_backward_pass(g.sdfg, g.state, ["y"], ["x", "w"])
    assert grads == {"x": "gradient_x", "w": "gradient_w"}
    expand_onnx_nodes(g.sdfg)
    dy = rng(62).standard_normal(want.shape).astype(np.float32)
    arrays = {"x": x.copy(), "w": w.copy(), "gradient_y": dy}
    em = run_state(g.sdfg, g.sdfg.states()[1], arrays)
    assert sorted(em.log) == ["dmlhip_conv2d_backward_data_f32", "dmlhip_conv2d_backward_weight_f32"]
    xt, wt = torch.tensor(x, dtype=torch.float64, requires_grad=True), torch.tensor(w, dtype=torch.float64, requires_grad=True)
    torch.nn.functional.conv1d(xt, wt, None, stride=stride, padding=pad, dilation=dil, groups=group).backward(
        torch.tensor(dy, dtype=torch.float64))
    assert_close(arrays["gradient_x"], xt.grad.numpy(), torch.float32, "conv1d dx", rtol=1e-5, atol=2e-6)
    assert_close(arrays["gradient_w"], wt.grad.numpy(), torch.float32, "conv1d dw", rtol=1e-5, atol=1e-5)


def test_exported_conv1d_module_imports_and_lowers():
    """torch.nn.Conv1d through the exporter, the importer's shape rule and the expansion, interpreted on the CPU."""
    from daceml_amd.onnx.onnx_importer import clean_onnx_name
    from daceml_amd.runtime import expand_onnx_nodes
    from daceml_amd.torch import DaceModule
    from tests.abi_emulator import run_state
    torch.manual_seed(4)
    net = torch.nn.Conv1d(6, 10, kernel_size=5, stride=2, padding=2, groups=2)
    x = torch.randn(3, 6, 50)
    model = DaceModule(net)._import((x, ))
    st = model.sdfg.states()[0]
    assert [n.schema.name for n in st.library_nodes()] == ["Conv"]
    expand_onnx_nodes(model.sdfg)
    names = [clean_onnx_name(n) for n in model.inputs]
    arrays = dict(zip(names, [x.numpy().copy(), net.weight.detach().numpy().copy(), net.bias.detach().numpy().copy()]))
    em = run_state(model.sdfg, st, arrays)
    assert em.log == ["dmlhip_conv2d_f32"]
    want = net.double()(x.double()).detach().numpy()
    assert_close(arrays[model.outputs[0]], want, torch.float32, "Conv1d module (emulated)", rtol=1e-5, atol=2e-6)


def test_shapes_that_are_not_a_1d_or_2d_convolution_are_refused():
    import daceml_amd.onnx as donnx
    from daceml_amd import graphs
    g = graphs.GraphBuilder("conv3d", torch.float32)
    ins = {"X": g.input("x", (1, 2, 4, 4, 4)), "W": g.input("w", (3, 2, 1, 1, 1))}
    g.output(g.node("Conv", ins, {"Y": (1, 3, 4, 4, 4)}, label="conv")["Y"], "y")
    with pytest.raises(donnx.NotApplicable):
        g.state.library_nodes()[0].expand(g.sdfg, g.state)
    g = graphs.GraphBuilder("conv1d_asym", torch.float32)
    ins = {"X": g.input("x", (1, 2, 9)), "W": g.input("w", (3, 2, 3))}
    g.output(g.node("Conv", ins, {"Y": (1, 3, 8)}, label="conv", pads=[1, 0])["Y"], "y")
    with pytest.raises(donnx.NotApplicable):
        g.state.library_nodes()[0].expand(g.sdfg, g.state)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("case", CASES)
def test_conv1d_on_gpu(case, dtype):
    """These sizes are served by the direct kernel (one thread per output element, every tap bounds-checked) and, for
    the 1 x 1 filter, by the contraction kernels."""
    from daceml_amd.runtime import CompiledSDFG
    n, c, l, m, k, stride, pad, dil, group, bias = case
    x, w, b, want = _data(*case, dtype=np.float16 if dtype == torch.float16 else np.float32)
    g = _graph(dtype, *case, out_l=want.shape[2])
    prog = CompiledSDFG(g.sdfg)
    y = torch.full(want.shape, float("nan"), dtype=dtype, device="cuda")
    args = {"x": dev(x), "w": dev(w), "y": y}
    if bias:
        args["b"] = dev(b)
    prog(**args)
    tol = dict(rtol=1e-5, atol=2e-6) if dtype == torch.float32 else dict(rtol=2e-2, atol=1e-2)
    assert_close(host(y), want, dtype, "conv1d %s" % (case, ), **tol)


@pytest.mark.gpu
def test_long_conv1d_on_gpu():
    from daceml_amd.runtime import CompiledSDFG
    case = (4, 32, 4096, 64, 5, 1, 2, 1, 1, True)
    x, w, b, want = _data(*case)
    g = _graph(torch.float32, *case, out_l=want.shape[2])
    prog = CompiledSDFG(g.sdfg)
    y = torch.full(want.shape, float("nan"), dtype=torch.float32, device="cuda")
    prog(x=dev(x), w=dev(w), b=dev(b), y=y)
    assert_close(host(y), want, torch.float32, "conv1d %s" % (case, ), rtol=1e-5, atol=1e-6 * (32 * 5) / 64)
