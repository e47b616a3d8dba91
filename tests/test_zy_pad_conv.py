"""A Pad with zeros in front of a Conv becomes the Conv's padding (PadConvFusion, pad_conv_fusion.py:13-104): the way
``nn.ZeroPad2d`` / ``F.pad`` + ``nn.Conv2d`` leave the exporter. What remains after the rewrite is an ordinary Conv
node, whose kernels have their own GPU tests. A Pad that does not fold (the padding differs between the two sides of
an axis, a fill value, other axes) runs on a kernel of its own; its reverse is a Pad with negated amounts. The calls
are interpreted on the CPU by tests/abi_emulator.py and compared with NumPy / PyTorch in double precision; the pad
kernel has a GPU test of its own."""
import numpy as np
import pytest
import torch

from tests.util import assert_close, dev, host


def _import(net, x):
    from daceml_amd.torch import DaceModule
    return DaceModule(net)._import((x, ))


def _run_emulated(model, net, x):
    from daceml_amd.onnx.onnx_importer import clean_onnx_name
    from daceml_amd.runtime import expand_onnx_nodes
    from tests.abi_emulator import run_state
    st = model.sdfg.states()[0]
    expand_onnx_nodes(model.sdfg)
    values = [x.numpy().copy()] + [p.detach().numpy().copy() for p in net.parameters()]
    arrays = dict(zip([clean_onnx_name(n) for n in model.inputs], values))
    em = run_state(model.sdfg, st, arrays)
    return em, arrays[model.outputs[0]]


@pytest.mark.parametrize("padding", [1, (2, 2, 1, 1)])
def test_exported_zero_pad_and_conv_become_one_conv(padding):
    """ZeroPad2d takes (left, right, top, bottom); the exporter computes the ONNX pads through a chain of shape
    arithmetic that the importer evaluates at import time."""
    torch.manual_seed(3)
    net = torch.nn.Sequential(torch.nn.ZeroPad2d(padding), torch.nn.Conv2d(4, 6, 3, stride=2))
    x = torch.randn(2, 4, 11, 12)
    model = _import(net, x)
    nodes = model.sdfg.states()[0].library_nodes()
    assert [n.schema.name for n in nodes] == ["Conv"]
    assert nodes[0].pads == ([1, 1, 1, 1] if padding == 1 else [1, 2, 1, 2])       # top, left, bottom, right
    em, got = _run_emulated(model, net, x)
    assert em.log == ["dmlhip_conv2d_f32"]
    assert_close(got, net.double()(x.double()).detach().numpy(), torch.float32, "pad + conv", rtol=1e-5, atol=2e-6)


def test_the_reference_test_module():
    """tests/transformation/test_pad_conv_fusion.py of the reference: ``F.pad(x, [2, 2])`` (the last axis only) in
    front of ``Conv2d(3, 6, 3)`` on a [4, 3, 24, 24] input - one rewrite, same output."""
    class Module(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.conv = torch.nn.Conv2d(3, 6, kernel_size=(3, 3))

        def forward(self, x):
            return self.conv(torch.nn.functional.pad(x, [2, 2]))

    from daceml_amd.torch import DaceModule
    from daceml_amd.transformation import fusion
    torch.manual_seed(11)
    net, x = Module(), torch.rand(4, 3, 24, 24)
    model = DaceModule(net, auto_optimize=False)._import((x, ))
    assert sorted(n.schema.name for n in model.sdfg.states()[0].library_nodes()) == ["Conv", "Pad"]
    assert fusion.fuse_pad_into_conv(model.sdfg) == 1
    nodes = model.sdfg.states()[0].library_nodes()
    assert [n.schema.name for n in nodes] == ["Conv"] and nodes[0].pads == [0, 2, 0, 2]
    _, got = _run_emulated(model, net, x)
    assert_close(got, net.double()(x.double()).detach().numpy(), torch.float32, "reference pad + conv module", rtol=1e-5,
                 atol=2e-6)


def test_padding_adds_to_the_padding_the_conv_has():
    torch.manual_seed(4)
    net = torch.nn.Sequential(torch.nn.ZeroPad2d(1), torch.nn.Conv2d(3, 5, 5, padding=1))
    x = torch.randn(1, 3, 8, 8)
    model = _import(net, x)
    nodes = model.sdfg.states()[0].library_nodes()
    assert [n.schema.name for n in nodes] == ["Conv"] and nodes[0].pads == [2, 2, 2, 2]
    _, got = _run_emulated(model, net, x)
    assert_close(got, net.double()(x.double()).detach().numpy(), torch.float32, "pad + padded conv", rtol=1e-5, atol=2e-6)


def test_exported_pad_and_conv1d():
    class Net(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.conv = torch.nn.Conv1d(4, 6, 3)

        def forward(self, x):
            return self.conv(torch.nn.functional.pad(x, (2, 2)))

    torch.manual_seed(5)
    net, x = Net(), torch.randn(2, 4, 30)
    model = _import(net, x)
    nodes = model.sdfg.states()[0].library_nodes()
    assert [n.schema.name for n in nodes] == ["Conv"] and nodes[0].pads == [2, 2]
    _, got = _run_emulated(model, net, x)
    assert_close(got, net.double()(x.double()).detach().numpy(), torch.float32, "pad + conv1d", rtol=1e-5, atol=2e-6)


def test_padding_that_differs_before_and_after_an_axis_stays_a_pad_node():
    """TensorFlow-style "same" padding of a strided convolution pads one side only: the convolution kernels take one
    padding per axis, so the Pad stays and runs as a kernel of its own in front of the unpadded Conv."""
    torch.manual_seed(6)
    net = torch.nn.Sequential(torch.nn.ZeroPad2d((0, 1, 0, 1)), torch.nn.Conv2d(4, 6, 3, stride=2))
    x = torch.randn(1, 4, 8, 8)
    model = _import(net, x)
    nodes = model.sdfg.states()[0].library_nodes()
    assert sorted(n.schema.name for n in nodes) == ["Conv", "Pad"]
    pad = [n for n in nodes if n.schema.name == "Pad"][0]
    assert pad.pads == [0, 0, 0, 0, 0, 0, 1, 1] and pad.mode == "constant" and pad.value == 0.0
    em, got = _run_emulated(model, net, x)
    assert em.log == ["dmlhip_pad_constant_f32", "dmlhip_conv2d_f32"]
    assert_close(got, net.double()(x.double()).detach().numpy(), torch.float32, "lopsided pad, conv", rtol=1e-5, atol=2e-6)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("shape,pads,value", [((2, 3, 5, 6), [0, 0, 1, 2, 0, 0, 0, 3], 0.0),
                                              ((4, 7), [1, 0, 2, 2], -2.5),
                                              ((3, 8, 5), [0, -2, 1, 0, -1, 0], 0.0)])
def test_pad_node_lowers_to_the_pad_entry_point(dtype, shape, pads, value):
    from daceml_amd import graphs
    from daceml_amd.runtime import expand_onnx_nodes
    from tests.abi_emulator import run_state
    npdt = np.float16 if dtype == torch.float16 else np.float32
    nd = len(shape)
    out = tuple(d + pads[i] + pads[nd + i] for i, d in enumerate(shape))
    g = graphs.GraphBuilder("pad", dtype)
    y = g.node("Pad", {"data": g.input("x", shape)}, {"output": out}, label="pad", pads=pads, value=value)["output"]
    g.output(y, "y")
    expand_onnx_nodes(g.sdfg)
    x = np.random.default_rng(8).standard_normal(shape).astype(npdt)
    arrays = {"x": x.copy(), "y": np.full(out, np.nan, npdt)}
    em = run_state(g.sdfg, g.state, arrays)
    assert em.log == ["dmlhip_pad_constant_" + ("f16" if dtype == torch.float16 else "f32")]
    crop = x[tuple(slice(max(-pads[i], 0), d - max(-pads[nd + i], 0)) for i, d in enumerate(shape))]
    want = np.pad(crop, [(max(pads[i], 0), max(pads[nd + i], 0)) for i in range(nd)], constant_values=npdt(value))
    assert np.array_equal(arrays["y"], want)


def test_pad_is_differentiated_by_cropping():
    """Pad -> Conv with a lopsided padding, differentiated: the Pad's reverse node is a Pad with negated amounts, and
    the input gradient equals autograd's."""
    from daceml_amd import graphs
    from daceml_amd.autodiff import add_backward_pass
    from daceml_amd.runtime import expand_onnx_nodes
    from tests.abi_emulator import run_sdfg
    g = graphs.GraphBuilder("pad_conv_train", torch.float32)
    p = g.node("Pad", {"data": g.input("x", (2, 3, 6, 6))}, {"output": (2, 3, 7, 8)}, label="pad",
               pads=[0, 0, 0, 2, 0, 0, 1, 0])["output"]
    y = g.node("Conv", {"X": p, "W": g.input("w", (4, 3, 3, 3))}, {"Y": (2, 4, 5, 6)}, label="conv", kernel_shape=[3, 3])["Y"]
    g.output(y, "y")
    add_backward_pass(g.sdfg, g.state, ["y"], ["x", "w"])
    back = [n for st in g.sdfg.states() for n in st.library_nodes() if n.label == "pad_backward"]
    assert len(back) == 1 and back[0].schema.name == "Pad" and back[0].pads == [0, 0, 0, -2, 0, 0, -1, 0]
    expand_onnx_nodes(g.sdfg)
    r = np.random.default_rng(9)
    x, w = r.standard_normal((2, 3, 6, 6)).astype(np.float32), (r.standard_normal((4, 3, 3, 3)) * 0.2).astype(np.float32)
    dy = r.standard_normal((2, 4, 5, 6)).astype(np.float32)
    arrays = {"x": x.copy(), "w": w.copy(), "gradient_y": dy.copy()}
    run_sdfg(g.sdfg, arrays)
    xt, wt = torch.tensor(x, dtype=torch.float64, requires_grad=True), torch.tensor(w, dtype=torch.float64, requires_grad=True)
    torch.nn.functional.conv2d(torch.nn.functional.pad(xt, (2, 0, 0, 1)), wt).backward(torch.tensor(dy, dtype=torch.float64))
    assert_close(arrays["gradient_x"], xt.grad.numpy(), torch.float32, "dx through pad", rtol=1e-5, atol=2e-6)
    assert_close(arrays["gradient_w"], wt.grad.numpy(), torch.float32, "dw behind pad", rtol=1e-5, atol=1e-5)


def _pad_conv_graph(pads, value=0.0, mode="constant", second_reader=False, conv_pads=None):
    from daceml_amd import graphs
    g = graphs.GraphBuilder("pad_conv", torch.float32)
    x = g.input("x", (1, 2, 6, 6))
    shape = tuple(d + pads[i] + pads[4 + i] for i, d in enumerate((1, 2, 6, 6)))
    p = g.node("Pad", {"data": x}, {"output": shape}, label="pad", pads=list(pads), value=value, mode=mode)["output"]
    cp = conv_pads or [0, 0, 0, 0]
    out = (1, 3, shape[2] + cp[0] + cp[2] - 2, shape[3] + cp[1] + cp[3] - 2)
    y = g.node("Conv", {"X": p, "W": g.input("w", (3, shape[1], 3, 3))}, {"Y": out}, label="conv", kernel_shape=[3, 3],
               pads=cp)["Y"]
    g.output(y, "y")
    if second_reader:
        g.output(g.node("Relu", {"X": p}, {"Y": shape}, label="relu")["Y"], "z")
    return g


def test_what_the_rewrite_refuses():
    from daceml_amd.transformation import fusion
    assert fusion.fuse_pad_into_conv(_pad_conv_graph([0, 0, 1, 2, 0, 0, 1, 2]).sdfg) == 1
    for kwargs in (dict(pads=[0, 0, 1, 1, 0, 0, 1, 1], value=1.0),                 # not zeros
                   dict(pads=[0, 0, 1, 1, 0, 0, 1, 1], mode="reflect"),
                   dict(pads=[0, 1, 1, 1, 0, 0, 1, 1]),                            # pads the channel axis
                   dict(pads=[1, 0, 1, 1, 0, 0, 1, 1]),                            # pads the batch axis
                   dict(pads=[0, 0, 1, 1, 0, 0, 1, 1], second_reader=True),        # the padded tensor is read elsewhere
                   dict(pads=[0, 0, 1, 1, 0, 0, 2, 1]),                            # top 1, bottom 2
                   dict(pads=[0, 0, 1, 1, 0, 0, 1, 1], conv_pads=[0, 0, 1, 0])):   # symmetric Pad, lopsided Conv
        g = _pad_conv_graph(**kwargs)
        assert fusion.fuse_pad_into_conv(g.sdfg) == 0, kwargs
        assert sorted(n.schema.name for n in g.state.library_nodes())[:2] == ["Conv", "Pad"]
    # a lopsided Pad that completes a lopsided Conv folds
    g = _pad_conv_graph(pads=[0, 0, 0, 1, 0, 0, 1, 0], conv_pads=[1, 0, 0, 1])
    assert fusion.fuse_pad_into_conv(g.sdfg) == 1
    assert g.state.library_nodes()[0].pads == [1, 1, 1, 1]


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("shape,pads,value", [((2, 3, 5, 6), [0, 0, 1, 2, 0, 0, 0, 3], 0.0), ((4, 7), [1, 0, 2, 2], -2.5),
                                              ((3, 8, 5), [0, -2, 1, 0, -1, 0], 0.0),
                                              ((96, 32, 112, 112), [0, 0, 0, 0, 0, 0, 1, 1], 0.0)])
def test_pad_on_gpu(dtype, shape, pads, value):
    from daceml_amd import kernels as K
    npdt = np.float16 if dtype == torch.float16 else np.float32
    nd = len(shape)
    x = np.random.default_rng(10).standard_normal(shape).astype(npdt)
    crop = x[tuple(slice(max(-pads[i], 0), d - max(-pads[nd + i], 0)) for i, d in enumerate(shape))]
    want = np.pad(crop, [(max(pads[i], 0), max(pads[nd + i], 0)) for i in range(nd)], constant_values=npdt(value))
    assert np.array_equal(host(K.pad(dev(x), pads, value)), want)
