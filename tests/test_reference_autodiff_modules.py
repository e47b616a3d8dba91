"""The modules of the reference's own autodiff test (tests/autodiff/torch/test_pytorch.py:76-262), differentiated here
the way its ``run_pytorch_module`` does (:13-73): the module's output is reduced with ``sum()`` or ``max()``, and the
gradient that reaches the input is compared with PyTorch's.

On the CPU the whole pipeline runs - export, import, the training form of the fusion pipeline, the backward pass, the
backward rewrites, expansion - and the calls of both states are interpreted by tests/abi_emulator.py; the gradient of
the reduction (ones, or a one at the maximum) is what the caller's autograd would hand over. On the GPU the same
modules run through ``DaceModule(backward=True)`` with the reference's tolerances; those tests compose kernels that run
on hardware, in shapes nothing else uses: a first run."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F
from torch import nn



class Simple(nn.Module):
    def forward(self, x):
        return torch.log(torch.sqrt(x))


class Repeated(nn.Module):
    def forward(self, x):
        return torch.sqrt(torch.sqrt(x))


class Softmax(nn.Module):
    def forward(self, x):
        return F.softmax(x, dim=1)


class ReshapeOnPath(nn.Module):
    def forward(self, x):
        reshaped = torch.reshape(x + 1, [3, 3])
        return torch.log(reshaped) + torch.reshape(torch.tensor([[3, 2, 1]], device=reshaped.device), [3])


class WeightsLN(nn.Module):
    def __init__(self):
        super().__init__()
        self.fc1 = nn.Linear(784, 120)
        self.fc2 = nn.Linear(120, 32)
        self.ln = nn.LayerNorm(32)
        self.fc3 = nn.Linear(32, 10)

    def forward(self, x):
        x = F.relu(self.fc1(x))
        x = F.relu(self.fc2(x))
        return self.fc3(self.ln(x))


class LN(nn.Module):
    def __init__(self):
        super().__init__()
        self.ln = nn.LayerNorm(3)

    def forward(self, x):
        return self.ln(x)


class Weights(nn.Module):
    def __init__(self):
        super().__init__()
        self.fc1 = nn.Linear(784, 120)
        self.fc2 = nn.Linear(120, 32)
        self.fc3 = nn.Linear(32, 10)

    def forward(self, x):
        return self.fc3(F.relu(self.fc2(F.relu(self.fc1(x)))))


class NestedSum(nn.Module):
    def __init__(self):
        super().__init__()
        self.fc1 = nn.Parameter(torch.rand(10, 10))

    def forward(self, x):
        return x * 2 + x @ self.fc1


class TransAdd(nn.Module):
    def forward(self, x):
        return torch.transpose((x + 1).reshape(4, 4), 1, 0)


class BatchedMatmul(nn.Module):
    def __init__(self):
        super().__init__()
        self.fc1 = nn.Parameter(torch.ones([10, 5, 3]))

    def forward(self, x):
        return self.fc1 @ x


class ScalarForwarding(nn.Module):
    def __init__(self):
        super().__init__()
        self.factor = nn.Parameter(torch.ones(()))

    def forward(self, x):
        return self.factor * x


class ScalarBuffer(nn.Module):
    def __init__(self):
        super().__init__()
        self.register_buffer("factor", torch.tensor(2))

    def forward(self, x):
        return self.factor * x


class BroadcastedMul(nn.Module):
    def forward(self, x):
        return x * x.sum(axis=0)


CASES = [("simple", Simple, {}), ("repeated", Repeated, {}), ("softmax", Softmax, dict(use_max=True)),
         ("reshape_on_memlet_path", ReshapeOnPath, dict(shape=(9, ))), ("weights_ln", WeightsLN, dict(shape=(4, 784))),
         ("layernorm", LN, dict(shape=(1, 3), use_max=True)), ("weights", Weights, dict(shape=(4, 784))),
         ("nested_gradient_summation", NestedSum, dict(shape=(4, 10))), ("trans_add", TransAdd, dict(shape=(16, ))),
         ("batched_matmul", BatchedMatmul, {}), ("scalar_forwarding", ScalarForwarding, {}),
         ("scalar_buffer", ScalarBuffer, {}), ("simple_broadcasted_mul", BroadcastedMul, {})]


def _emulated_input_gradient(module, shape=(3, 5), use_max=False):
    from daceml_amd.autodiff import add_backward_pass
    from daceml_amd.onnx.onnx_importer import clean_onnx_name
    from daceml_amd.runtime import expand_onnx_nodes
    from daceml_amd.torch import DaceModule
    from daceml_amd.transformation import fusion
    from tests.abi_emulator import run_sdfg
    torch.manual_seed(0)
    x = torch.rand(*shape, dtype=torch.float32)
    xt = x.clone().requires_grad_(True)
    out = module(xt)
    (out.max() if use_max else out.sum()).backward()
    model = DaceModule(module, backward=True, auto_optimize=False)._import((x, ))
    sdfg, st = model.sdfg, model.sdfg.states()[0]
    fusion.auto_optimize(sdfg, training=True)
    names = [clean_onnx_name(n) for n in model.inputs]
    add_backward_pass(sdfg, st, list(model.outputs), names[:1])
    fusion.optimize_backward(sdfg)
    expand_onnx_nodes(sdfg)
    tensors = dict(module.named_parameters())
    tensors.update(dict(module.named_buffers()))
    arrays = {names[0]: x.numpy().copy()}
    for n in model.inputs[1:]:
        arrays[clean_onnx_name(n)] = tensors[n].detach().numpy().copy()
    g = torch.zeros_like(out)
    if use_max:
        g.view(-1)[out.argmax()] = 1.0
    else:
        g[...] = 1.0
    arrays["gradient_" + model.outputs[0]] = g.numpy().copy()
    run_sdfg(sdfg, arrays)
    return arrays["gradient_" + names[0]], xt.grad.numpy()


@pytest.mark.parametrize("name", [c[0] for c in CASES])
def test_reference_autodiff_module_lowers_correctly(name):
    _, make, kwargs = next(c for c in CASES if c[0] == name)
    got, want = _emulated_input_gradient(make(), **kwargs)
    np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-5)


@pytest.mark.gpu
@pytest.mark.parametrize("name", [c[0] for c in CASES])
def test_reference_autodiff_module_on_gpu(name):
    from daceml_amd.torch import DaceModule
    _, make, kwargs = next(c for c in CASES if c[0] == name)
    torch.manual_seed(0)
    module = make().cuda()
    shape, use_max = kwargs.get("shape", (3, 5)), kwargs.get("use_max", False)
    value = torch.rand(*shape, dtype=torch.float32).cuda()
    pytorch_input = value.clone().requires_grad_(True)
    out = module(pytorch_input)
    (out.max() if use_max else out.sum()).backward()
    dace_input = value.clone().requires_grad_(True)
    out = DaceModule(module, backward=True)(dace_input)
    (out.max() if use_max else out.sum()).backward()
    torch.testing.assert_close(dace_input.grad, pytorch_input.grad, rtol=1e-4, atol=1e-3)   # the reference's tolerances


# ----------------------------------------------------------------------------- tests/torch/test_conv2d.py
class TwoConvs(nn.Module):
    def __init__(self):
        super().__init__()
        self.conv1 = nn.Conv2d(1, 4, 3)
        self.conv2 = nn.Conv2d(4, 4, 3)

    def forward(self, x):
        x = F.relu(self.conv1(x))
        return F.relu(self.conv2(x))


def test_reference_conv2d_model_lowers_correctly():
    """tests/torch/test_conv2d.py:12-86: Conv, Relu, Conv, Relu on a [1, 1, 8, 8] input - output to 1e-6 as the reference
    asserts, and the input gradient for a given output gradient (its cuDNN variant)."""
    from daceml_amd.autodiff import add_backward_pass
    from daceml_amd.onnx.onnx_importer import clean_onnx_name
    from daceml_amd.runtime import expand_onnx_nodes
    from daceml_amd.torch import DaceModule, dace_module
    from tests.abi_emulator import run_sdfg
    torch.manual_seed(0)
    net = TwoConvs()
    x, dy = torch.rand(1, 1, 8, 8), torch.rand(1, 4, 4, 4)

    @dace_module(sdfg_name="decorated")
    class Decorated(TwoConvs):
        pass

    assert isinstance(Decorated(), DaceModule)                      # the decorator form the reference's test also builds
    model = DaceModule(net, backward=True, sdfg_name="wrapped")._import((x, ))
    sdfg = model.sdfg
    names = [clean_onnx_name(n) for n in model.inputs]
    add_backward_pass(sdfg, sdfg.states()[0], list(model.outputs), names[:1])
    expand_onnx_nodes(sdfg)
    arrays = dict(zip(names, [x.numpy().copy()] + [p.detach().numpy().copy() for p in net.parameters()]))
    arrays["gradient_" + model.outputs[0]] = dy.numpy().copy()
    run_sdfg(sdfg, arrays)
    xt = x.clone().requires_grad_(True)
    out = net(xt)
    out.backward(dy)
    assert np.allclose(arrays[model.outputs[0]], out.detach().numpy(), atol=1e-6)
    np.testing.assert_allclose(arrays["gradient_" + names[0]], xt.grad.numpy(), rtol=1e-5, atol=1e-6)


@pytest.mark.gpu
def test_reference_conv2d_model_on_gpu():
    from daceml_amd.torch import DaceModule
    torch.manual_seed(0)
    net = TwoConvs().cuda()
    value, dy = torch.rand(1, 1, 8, 8).cuda(), torch.rand(1, 4, 4, 4).cuda()
    dace_inputs, torch_inputs = value.clone().requires_grad_(True), value.clone().requires_grad_(True)
    dace_output = DaceModule(net, backward=True)(dace_inputs)
    dace_output.backward(dy)
    torch_output = net(torch_inputs)
    torch_output.backward(dy)
    torch.testing.assert_close(dace_output, torch_output, rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(dace_inputs.grad, torch_inputs.grad, rtol=1e-5, atol=1e-6)


# ----------------------------------------------------------------------------- tests/torch/test_img_op_implementations.py
def _emulated_forward(net, x, training):
    from daceml_amd.onnx.onnx_importer import clean_onnx_name
    from daceml_amd.runtime import expand_onnx_nodes
    from daceml_amd.torch import DaceModule
    from tests.abi_emulator import run_state
    model = DaceModule(net, training=training)._import((x, ))
    st = model.sdfg.states()[0]
    expand_onnx_nodes(model.sdfg)
    tensors = dict(net.named_parameters())
    tensors.update(dict(net.named_buffers()))
    arrays = {clean_onnx_name(model.inputs[0]): x.numpy().copy()}
    for n in model.inputs[1:]:
        arrays[clean_onnx_name(n)] = tensors[n].detach().numpy().copy()
    run_state(model.sdfg, st, arrays)
    return model, arrays


def test_reference_batchnorm_module_lowers_correctly():
    """test_bn (:9-29): ``BatchNorm2d(64)`` in training mode on [1, 64, 60, 60] - output and both running statistics."""
    from daceml_amd.onnx.onnx_importer import clean_onnx_name
    torch.manual_seed(0)
    x = torch.rand(1, 64, 60, 60)
    pt_model, dace_model = nn.BatchNorm2d(64), nn.BatchNorm2d(64)
    dace_model.load_state_dict(pt_model.state_dict())
    model, arrays = _emulated_forward(dace_model, x, training=True)
    want = pt_model(x)
    np.testing.assert_allclose(arrays[model.outputs[0]], want.detach().numpy(), rtol=1e-4, atol=1e-5)
    # the running statistics come back either in place or as further outputs, depending on what reads them
    written = {n: a for n, a in arrays.items() if a.shape == (64, )}
    assert any(np.allclose(a, pt_model.running_mean.numpy(), rtol=1e-4, atol=1e-6) for a in written.values())
    assert any(np.allclose(a, pt_model.running_var.numpy(), rtol=1e-4, atol=1e-6) for a in written.values())
    assert clean_onnx_name("running_mean") in arrays


def test_reference_global_average_pool_module_lowers_correctly():
    """test_global_avg_pool (:32-42): ``AdaptiveAvgPool2d(1)`` on [1, 64, 60, 60]."""
    torch.manual_seed(0)
    x = torch.rand(1, 64, 60, 60)
    model, arrays = _emulated_forward(nn.AdaptiveAvgPool2d(1), x, training=True)
    np.testing.assert_allclose(arrays[model.outputs[0]], nn.AdaptiveAvgPool2d(1)(x).numpy(), rtol=1e-5, atol=1e-6)


# ----------------------------------------------------------------------------- tests/torch/test_reshape.py, test_multi_output.py
def test_reference_reshape_module_lowers_correctly():
    """test_reshape_module (:20-35): ``x.reshape([5, 5])`` of a [25] input, without the fusion pipeline."""
    from daceml_amd.torch import DaceModule

    class Model(nn.Module):
        def forward(self, x):
            return x.reshape([5, 5])

    from daceml_amd.onnx.onnx_importer import clean_onnx_name
    from daceml_amd.runtime import expand_onnx_nodes
    from tests.abi_emulator import run_state
    x = torch.rand([25])
    model = DaceModule(Model(), auto_optimize=False, dummy_inputs=None)._import((x, ))
    st = model.sdfg.states()[0]
    expand_onnx_nodes(model.sdfg)
    arrays = {clean_onnx_name(model.inputs[0]): x.numpy().copy()}
    run_state(model.sdfg, st, arrays)
    np.testing.assert_array_equal(arrays[model.outputs[0]], x.numpy().reshape(5, 5))


def test_reference_two_input_two_output_module_lowers_correctly():
    """tests/torch/test_multi_output.py (:11-37): ``(x + y, x * y)`` style modules with several inputs and outputs."""
    from daceml_amd.onnx.onnx_importer import clean_onnx_name
    from daceml_amd.runtime import expand_onnx_nodes
    from daceml_amd.torch import DaceModule
    from tests.abi_emulator import run_state

    class Model(nn.Module):
        def forward(self, x, y):
            return x + y, x * y

    x, y = torch.rand(5, 10), torch.rand(5, 10)
    model = DaceModule(Model())._import((x, y))
    st = model.sdfg.states()[0]
    expand_onnx_nodes(model.sdfg)
    arrays = dict(zip([clean_onnx_name(n) for n in model.inputs], [x.numpy().copy(), y.numpy().copy()]))
    run_state(model.sdfg, st, arrays)
    np.testing.assert_allclose(arrays[model.outputs[0]], (x + y).numpy(), rtol=1e-6)
    np.testing.assert_allclose(arrays[model.outputs[1]], (x * y).numpy(), rtol=1e-6)
