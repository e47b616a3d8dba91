"""MaxPool (PureMaxPool2D, img_op_implementations.py:28-161; DefaultMaxPoolBackward, onnx_ops.py:284-335) and the network
of the reference's tests/torch/test_lenet.py, which needs it: Conv, Relu, MaxPool twice, three Linear layers, LogSoftmax.

Host side: lowering and the emitted calls interpreted by tests/abi_emulator.py against the oracle / PyTorch; the GPU
tests run the pool kernels and the network on them."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F
from torch import nn

from oracle import ops as O
from tests.util import assert_close, dev, host

CASES = [((2, 3, 8, 8), [2, 2], [2, 2]), ((1, 2, 9, 7), [3, 3], [2, 2]), ((2, 1, 7, 10), [3, 2], [1, 3]),
         ((1, 4, 13, 13), [2, 2], [2, 2])]


def _graph(dtype, shape, kernel, strides, backward):
    from daceml_amd import graphs
    from daceml_amd.autodiff import add_backward_pass
    n, c, h, w = shape
    out = (n, c, (h - kernel[0]) // strides[0] + 1, (w - kernel[1]) // strides[1] + 1)
    g = graphs.GraphBuilder("maxpool", dtype)
    y = g.node("MaxPool", {"X": g.input("x", shape)}, {"Y": out}, label="pool", kernel_shape=kernel, strides=strides)["Y"]
    g.output(y, "y")
    if backward:
        add_backward_pass(g.sdfg, g.state, ["y"], ["x"])
    return g, out


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("shape,kernel,strides", CASES)
def test_maxpool_node_and_its_reverse_lower_correctly(dtype, shape, kernel, strides):
    from daceml_amd.runtime import expand_onnx_nodes
    from tests.abi_emulator import run_sdfg
    npdt = np.float16 if dtype == torch.float16 else np.float32
    g, out = _graph(dtype, shape, kernel, strides, backward=True)
    assert [n.schema.name for n in g.sdfg.states()[1].library_nodes()] == ["MaxPoolGrad"]
    expand_onnx_nodes(g.sdfg)
    r = np.random.default_rng(12)
    x = np.round(r.standard_normal(shape) * 2).astype(npdt)           # equal maxima are common
    dy = r.standard_normal(out).astype(npdt)
    arrays = {"x": x.copy(), "gradient_y": dy.copy()}
    sfx = "f16" if dtype == torch.float16 else "f32"
    assert run_sdfg(g.sdfg, arrays) == ["dmlhip_maxpool2d_" + sfx, "dmlhip_maxpool2d_backward_" + sfx]
    assert np.array_equal(arrays["y"], O.maxpool2d(x.astype(np.float64), kernel, strides).astype(npdt))
    want = O.maxpool2d_backward(x.astype(np.float64), dy.astype(np.float64), kernel, strides)
    assert_close(arrays["gradient_x"], want, dtype, "MaxPool reverse", **({} if dtype == torch.float16 else
                                                                          dict(rtol=1e-6, atol=1e-6)))


def test_maxpool_refuses_what_the_reference_refuses():
    """forward_can_be_applied of PureMaxPool2D (:31-61): padding, dilation, ceil_mode, the Indices output."""
    import daceml_amd.onnx as donnx
    from daceml_amd import graphs
    for attrs in (dict(pads=[1, 1, 1, 1]), dict(dilations=[2, 2]), dict(ceil_mode=1), dict(storage_order=1),
                  dict(auto_pad="SAME_UPPER")):
        g = graphs.GraphBuilder("maxpool_refused", torch.float32)
        y = g.node("MaxPool", {"X": g.input("x", (1, 1, 8, 8))}, {"Y": (1, 1, 4, 4)}, label="pool", kernel_shape=[2, 2],
                   strides=[2, 2], **attrs)["Y"]
        g.output(y, "y")
        with pytest.raises(donnx.NotApplicable):
            g.state.library_nodes()[0].expand(g.sdfg, g.state)


class LeNet(nn.Module):
    def __init__(self):
        super().__init__()
        self.conv1 = nn.Conv2d(1, 6, (3, 3))
        self.conv2 = nn.Conv2d(6, 16, (3, 3))
        self.fc1 = nn.Linear(16 * 6 * 6, 120)
        self.fc2 = nn.Linear(120, 84)
        self.fc3 = nn.Linear(84, 10)

    def forward(self, x):
        x = F.max_pool2d(F.relu(self.conv1(x)), 2)
        x = F.max_pool2d(F.relu(self.conv2(x)), 2)
        x = x.view(-1, 16 * 6 * 6)
        x = F.relu(self.fc1(x))
        x = F.relu(self.fc2(x))
        x = self.fc3(x)
        return F.log_softmax(x, dim=1)


def test_lenet_forward_and_training_step_lower_correctly():
    """tests/torch/test_lenet.py: ``torch.rand(8, 1, 32, 32)`` through LeNet; here also a training step under NLLLoss."""
    from daceml_amd.autodiff import add_backward_pass
    from daceml_amd.onnx.onnx_importer import clean_onnx_name
    from daceml_amd.runtime import expand_onnx_nodes
    from daceml_amd.torch import DaceModule
    from daceml_amd.transformation import fusion
    from tests.abi_emulator import run_state
    torch.manual_seed(0)
    net = LeNet()
    x, labels = torch.rand(8, 1, 32, 32), torch.randint(0, 10, [8])
    model = DaceModule(net, backward=True, auto_optimize=False)._import((x, ))
    sdfg, st = model.sdfg, model.sdfg.states()[0]
    names = [n.schema.name for n in st.library_nodes()]
    assert names.count("MaxPool") == 2 and names.count("LogSoftmax") == 1 and names.count("Conv") == 2
    fusion.auto_optimize(sdfg, training=True)
    trained = list(dict(net.named_parameters()))
    add_backward_pass(sdfg, st, list(model.outputs), [clean_onnx_name(n) for n in trained])
    fusion.optimize_backward(sdfg)
    expand_onnx_nodes(sdfg)
    tensors = dict(net.named_parameters())
    arrays = {clean_onnx_name(model.inputs[0]): x.numpy().copy()}
    for n in model.inputs[1:]:
        arrays[clean_onnx_name(n)] = tensors[n].detach().numpy().copy()
    fwd, bwd = sdfg.states()
    run_state(sdfg, fwd, arrays)
    ref = LeNet().double()
    ref.load_state_dict({k: v.double() for k, v in net.state_dict().items()})
    want = ref(x.double())
    assert_close(arrays[model.outputs[0]], want.detach().numpy(), torch.float32, "LeNet output", rtol=1e-5, atol=1e-5)
    out = torch.tensor(arrays[model.outputs[0]], requires_grad=True)
    nn.NLLLoss()(out, labels).backward()
    arrays["gradient_" + model.outputs[0]] = out.grad.numpy().copy()
    run_state(sdfg, bwd, arrays)
    nn.NLLLoss()(want, labels).backward()
    for pname, p in ref.named_parameters():
        w = p.grad.numpy()
        assert_close(arrays["gradient_" + clean_onnx_name(pname)], w, torch.float32, "LeNet gradient of " + pname, rtol=1e-4,
                     atol=1e-6 * max(1.0, float(np.abs(w).max()) * 10))


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("shape,kernel,strides", CASES + [((64, 16, 112, 112), [2, 2], [2, 2])])
def test_maxpool_on_gpu(dtype, shape, kernel, strides):
    from daceml_amd import kernels as K
    g = torch.Generator().manual_seed(13)
    x = torch.round(torch.randn(shape, generator=g) * 2).to(dtype).cuda()
    xt = x.double().requires_grad_(True)
    want = F.max_pool2d(xt, kernel, strides)
    dy = torch.randn(want.shape, generator=g).to(dtype).cuda()
    want.backward(dy.double())
    assert torch.equal(K.max_pool2d(x, kernel, strides), want.detach().to(dtype))
    torch.testing.assert_close(K.max_pool2d_backward(x, dy, kernel, strides).double(), xt.grad,
                               **(dict(rtol=2e-2, atol=1e-2) if dtype == torch.float16 else dict(rtol=1e-6, atol=1e-6)))


@pytest.mark.gpu
def test_lenet_on_gpu():
    from daceml_amd.torch import DaceModule
    torch.manual_seed(0)
    net = LeNet().cuda()
    x = torch.rand(8, 1, 32, 32).cuda()
    torch.testing.assert_close(DaceModule(net)(x.clone()), net(x.clone()), rtol=1e-5, atol=1e-5)
