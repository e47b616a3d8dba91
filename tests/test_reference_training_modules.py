"""The two networks of the reference's training test (tests/autodiff/torch/test_training.py:76-131) - an MNIST-sized
classifier ending in LayerNorm and LogSoftmax, and a HuggingFace ``BertLayer`` (relu) under a token-sum LogSoftmax -
under ``NLLLoss``: loss value, the gradient of every parameter, and the parameters after one SGD step against PyTorch.

On the CPU the graphs run through export, import, fusion, autodiff and expansion and their calls are interpreted by
tests/abi_emulator.py; the loss and its gradient are computed by PyTorch on the emulated output, as the caller's
autograd would. The GPU forms run ``DaceModule(backward=True)`` as the reference's ``training_step`` does and are a
first run on hardware."""
import numpy as np
import pytest
import torch
from torch import nn, optim

from tests.util import assert_close


def _mnist():
    return nn.Sequential(nn.Linear(784, 128), nn.ReLU(), nn.Linear(128, 64), nn.ReLU(), nn.Linear(64, 10),
                         nn.LayerNorm(10), nn.LogSoftmax(dim=1))


class BertTokenSoftmaxClf(nn.Module):
    def __init__(self):
        super().__init__()
        from transformers import BertConfig
        from transformers.models.bert.modeling_bert import BertLayer
        self.bert = BertLayer(BertConfig(hidden_act="relu")).eval()
        self.sm = nn.LogSoftmax(dim=-1)

    def forward(self, x):
        out = self.bert(x)          # a tuple in the transformers release the reference used, the tensor itself later
        embs = out[0] if isinstance(out, tuple) else out
        return self.sm(embs.sum(dim=-1))


def _cases():
    torch.manual_seed(0)
    yield "mnist", _mnist, (torch.randn(64, 784), torch.randint(0, 10, [64], dtype=torch.long))
    yield "bert", BertTokenSoftmaxClf, (torch.randn([2, 512, 768]), torch.tensor([0, 123], dtype=torch.long))


def _emulated_training_step(net, x, labels):
    from daceml_amd.autodiff import add_backward_pass
    from daceml_amd.onnx.onnx_importer import clean_onnx_name
    from daceml_amd.runtime import expand_onnx_nodes
    from daceml_amd.torch import DaceModule
    from daceml_amd.transformation import fusion
    from tests.abi_emulator import run_state
    model = DaceModule(net, backward=True, auto_optimize=False)._import((x, ))
    sdfg, st = model.sdfg, model.sdfg.states()[0]
    fusion.auto_optimize(sdfg, training=True)
    tensors = dict(net.named_parameters())
    tensors.update(dict(net.named_buffers()))
    trained = [n for n in model.inputs[1:] if n in dict(net.named_parameters())]
    add_backward_pass(sdfg, st, list(model.outputs), [clean_onnx_name(n) for n in trained])
    fusion.optimize_backward(sdfg)
    expand_onnx_nodes(sdfg)
    arrays = {clean_onnx_name(model.inputs[0]): x.numpy().copy()}
    for n in model.inputs[1:]:
        arrays[clean_onnx_name(n)] = tensors[n].detach().numpy().copy()
    fwd, bwd = sdfg.states()
    run_state(sdfg, fwd, arrays)
    out = torch.tensor(arrays[model.outputs[0]], requires_grad=True)
    loss = nn.NLLLoss()(out, labels)
    loss.backward()
    arrays["gradient_" + model.outputs[0]] = out.grad.numpy().copy()
    run_state(sdfg, bwd, arrays)
    return loss.item(), {n: arrays["gradient_" + clean_onnx_name(n)] for n in trained}


@pytest.mark.parametrize("name", ["mnist", "bert"])
def test_training_step_lowers_correctly(name):
    _, make, (x, labels) = next(c for c in _cases() if c[0] == name)
    torch.manual_seed(1)
    net = make()
    ref = make().double()
    ref.load_state_dict({k: v.double() for k, v in net.state_dict().items()})
    loss = nn.NLLLoss()(ref(x.double()), labels)
    loss.backward()
    got_loss, grads = _emulated_training_step(net, x, labels)
    assert abs(got_loss - loss.item()) / abs(loss.item()) < 1e-5             # the reference's bound on the loss
    want = dict(ref.named_parameters())
    assert set(grads) == set(want)
    for pname, g in grads.items():
        w = want[pname].grad.numpy()
        assert_close(g, w, torch.float32, "%s: gradient of %s" % (name, pname), rtol=1e-4,
                     atol=1e-5 * max(1.0, float(np.abs(w).max())))


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["mnist", "bert"])
def test_training_step_on_gpu(name):
    """``training_step`` of the reference (:17-73): loss, parameter gradients, parameters after an SGD step."""
    from daceml_amd.torch import DaceModule
    _, make, (x, labels) = next(c for c in _cases() if c[0] == name)
    torch.manual_seed(1)
    pt_model = make().cuda()
    dace_model = make().cuda()
    dace_model.load_state_dict(pt_model.state_dict())
    dace_model = DaceModule(dace_model, backward=True)
    x, labels = x.cuda(), labels.cuda()
    pt_loss = nn.NLLLoss()(pt_model(x), labels)
    dace_loss = nn.NLLLoss()(dace_model(x), labels)
    assert abs(pt_loss.item() - dace_loss.item()) / pt_loss.item() < 1e-5
    pt_loss.backward()
    dace_loss.backward()
    for (pname, pt_param), (dname, dace_param) in zip(pt_model.named_parameters(), dace_model.named_parameters()):
        assert "model." + pname == dname
        torch.testing.assert_close(dace_param.grad, pt_param.grad, rtol=1e-4, atol=1e-5)
    optim.SGD(pt_model.parameters(), lr=0.001).step()
    optim.SGD(dace_model.parameters(), lr=0.001).step()
    for (pname, pt_param), (dname, dace_param) in zip(pt_model.named_parameters(), dace_model.named_parameters()):
        torch.testing.assert_close(dace_param.detach(), pt_param.detach(), rtol=1e-4, atol=1e-5)
