"""Wrapper cases of the reference's autodiff tests that the other test files do not have:
tests/autodiff/torch/test_multi_output_ad.py (two outputs, ``backward`` called on each in turn with ``retain_graph``) and
tests/autodiff/torch/test_dont_compute_input_grads.py (``inputs_to_skip``: the parameter's gradient is computed, the
input's is not part of the backward graph at all)."""
import numpy as np
import pytest
import torch
from torch import nn



class TwoOutputs(nn.Module):
    def forward(self, x):
        return x + 1, x * 2


class OneWeight(nn.Module):
    def __init__(self):
        super().__init__()
        self.fc1 = nn.Parameter(torch.rand(10, 10))

    def forward(self, x):
        return x @ self.fc1


def test_a_skipped_input_has_no_gradient_in_the_backward_graph():
    """test_dont_compute_input_grads.py:46-47: the backward graph ends in one array - the parameter's gradient."""
    from daceml_amd.autodiff import add_backward_pass
    from daceml_amd.onnx.onnx_importer import clean_onnx_name
    from daceml_amd.runtime import expand_onnx_nodes
    from daceml_amd.sdfg import AccessNode
    from daceml_amd.torch import DaceModule
    from tests.abi_emulator import run_sdfg
    torch.manual_seed(0)
    net, x, dy = OneWeight(), torch.rand(8, 10), torch.rand(8, 10)
    model = DaceModule(net, backward=True, inputs_to_skip=["0"])._import((x, ))
    names = [clean_onnx_name(n) for n in model.inputs]
    add_backward_pass(model.sdfg, model.sdfg.states()[0], list(model.outputs), names[1:])
    bst = model.sdfg.states()[1]
    sinks = [n for n in bst.nodes() if isinstance(n, AccessNode) and not bst.out_edges(n)]
    assert [n.data for n in sinks] == ["gradient_" + names[1]]
    expand_onnx_nodes(model.sdfg)
    arrays = {names[0]: x.numpy().copy(), names[1]: net.fc1.detach().numpy().copy(),
              "gradient_" + model.outputs[0]: dy.numpy().copy()}
    run_sdfg(model.sdfg, arrays)
    (x @ net.fc1).backward(dy)
    np.testing.assert_allclose(arrays["gradient_" + names[1]], net.fc1.grad.numpy(), rtol=1e-5, atol=1e-6)


@pytest.mark.gpu
def test_skip_input_grads_on_gpu():
    from daceml_amd.torch import DaceModule
    torch.manual_seed(0)
    pt_module = OneWeight().cuda()
    dace_module = OneWeight().cuda()
    dace_module.load_state_dict(pt_module.state_dict())
    value, dy = torch.rand(8, 10).cuda(), torch.rand(8, 10).cuda()
    wrapped = DaceModule(dace_module, backward=True, inputs_to_skip=["0"])
    dace_output, pt_output = wrapped(value.clone()), pt_module(value.clone())
    torch.testing.assert_close(dace_output, pt_output)
    dace_output.backward(dy)
    pt_output.backward(dy)
    torch.testing.assert_close(wrapped.model.fc1.grad, pt_module.fc1.grad)


@pytest.mark.gpu
def test_backward_called_per_output_on_gpu():
    """test_multi_output_ad.py:8-48: each output's ``backward`` in turn; the input gradient accumulates."""
    from daceml_amd.torch import DaceModule
    torch.manual_seed(0)
    module = TwoOutputs().cuda()
    value = torch.rand(5, 10).cuda()
    pytorch_input, dace_input = value.clone().requires_grad_(True), value.clone().requires_grad_(True)
    dy = torch.randn(5, 10).cuda()
    y1, y2 = module(pytorch_input)
    y1.backward(dy)
    y2.backward(dy)
    d1, d2 = DaceModule(module, backward=True)(dace_input)
    d1.backward(dy.clone(), retain_graph=True)
    d2.backward(dy.clone())
    torch.testing.assert_close(dace_input.grad, pytorch_input.grad)
