"""``torch.nn.MultiheadAttention`` through the wrapper, as tests/torch/test_attn.py of the reference runs it (packed
q / k / v projection weight, both outputs: the attention result and the head-averaged weights).

The exporter slices the packed weight three times; the importer turns a Slice with known bounds into a view of its
input (no node, no copy), and the backward pass pads the gradient of each slice back into a contribution shaped like
the packed weight. Host side: the graph is lowered and its calls are interpreted on the CPU by tests/abi_emulator.py,
against PyTorch in double precision. The GPU tests run the forward pass (operand pointers offset into the packed
weight) and a training step (which also runs the constant-pad kernel) at the shapes of the reference's test."""
from collections import Counter

import numpy as np
import pytest
import torch

from tests.util import assert_close


def _reference(pt, tensors, grads=None):
    ptd = torch.nn.MultiheadAttention(pt.embed_dim, pt.num_heads, bias=pt.in_proj_bias is not None).double()
    ptd.load_state_dict({k: v.double() for k, v in pt.state_dict().items()})
    ins = [t.double().requires_grad_(grads is not None) for t in tensors]
    outs = ptd(*ins)
    if grads is None:
        return [o.detach().numpy() for o in outs], None
    torch.autograd.backward(list(outs), [torch.tensor(g, dtype=torch.float64) for g in grads])
    return [o.detach().numpy() for o in outs], [t.grad.numpy() for t in ins] + [p.grad.numpy() for p in ptd.parameters()]


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
def test_multihead_attention_forward_lowers_correctly(dtype):
    from daceml_amd.onnx.onnx_importer import clean_onnx_name
    from daceml_amd.runtime import expand_onnx_nodes
    from daceml_amd.torch import DaceModule
    from tests.abi_emulator import run_state
    torch.manual_seed(0)
    n, heads, s, b = 256, 4, 128, 2
    q, k, v = (torch.randn(s, b, n).to(dtype) for _ in range(3))
    pt = torch.nn.MultiheadAttention(n, heads, bias=False).to(dtype)
    model = DaceModule(pt)._import((q, k, v))
    sdfg, st = model.sdfg, model.sdfg.states()[0]
    # the three slices of the packed weight are views at offsets 0, n*n, 2*n*n; no Slice node, no copy
    views = sorted(d.view_offset for d in sdfg.arrays.values() if d.view_of == "in_proj_weight" and d.shape == (n, n))
    assert views[:3] == [0, n * n, 2 * n * n]
    assert Counter(nd.schema.name for nd in st.library_nodes())["Einsum"] == 6
    expand_onnx_nodes(sdfg)
    names = [clean_onnx_name(x) for x in model.inputs]
    arrays = dict(zip(names, [t.numpy().copy() for t in (q, k, v)] + [p.detach().numpy().copy() for p in pt.parameters()]))
    run_state(sdfg, st, arrays)
    want, _ = _reference(pt, (q, k, v))
    for out, w in zip(model.outputs, want):
        assert_close(arrays[out], w, dtype, "MultiheadAttention " + out, **({} if dtype == torch.float16 else
                                                                           dict(rtol=1e-5, atol=2e-6)))


def test_multihead_attention_training_step_lowers_correctly():
    from daceml_amd.autodiff import add_backward_pass
    from daceml_amd.onnx.onnx_importer import clean_onnx_name
    from daceml_amd.runtime import expand_onnx_nodes
    from daceml_amd.torch import DaceModule
    from daceml_amd.transformation import fusion
    from tests.abi_emulator import run_sdfg
    torch.manual_seed(1)
    n, heads, s, b = 128, 2, 40, 2
    q, k, v = (torch.randn(s, b, n) for _ in range(3))
    pt = torch.nn.MultiheadAttention(n, heads, bias=False)
    model = DaceModule(pt, backward=True, auto_optimize=False)._import((q, k, v))
    sdfg, st = model.sdfg, model.sdfg.states()[0]
    fusion.auto_optimize(sdfg, training=True)
    names = [clean_onnx_name(x) for x in model.inputs]
    add_backward_pass(sdfg, st, list(model.outputs), names)
    fusion.optimize_backward(sdfg)
    back = Counter(nd.schema.name for nd in sdfg.states()[1].library_nodes())
    assert back["Pad"] == 3 and back["Sum"] >= 1      # three slice gradients padded to the packed shape and summed
    expand_onnx_nodes(sdfg)
    r = np.random.default_rng(2)
    arrays = dict(zip(names, [t.numpy().copy() for t in (q, k, v)] + [p.detach().numpy().copy() for p in pt.parameters()]))
    grads = [r.standard_normal(sdfg.arrays[o].shape).astype(np.float32) for o in model.outputs]
    for o, g in zip(model.outputs, grads):
        arrays["gradient_" + o] = g.copy()
    run_sdfg(sdfg, arrays)
    outs, want = _reference(pt, (q, k, v), grads)
    for o, w in zip(model.outputs, outs):
        assert_close(arrays[o], w, torch.float32, o, rtol=1e-5, atol=2e-6)
    for name, w in zip(names, want):
        assert_close(arrays["gradient_" + name], w, torch.float32, "gradient of " + name, rtol=1e-4,
                     atol=2e-6 * max(1.0, float(np.abs(w).max())))


def test_the_wrapper_asks_for_the_gradient_of_a_weight_that_is_read_through_views_only():
    from daceml_amd.torch import DaceModule
    torch.manual_seed(5)
    n, heads, s, b = 128, 2, 24, 2
    q, k, v = (torch.randn(s, b, n) for _ in range(3))
    dm = DaceModule(torch.nn.MultiheadAttention(n, heads, bias=False), backward=True)
    need = dm._inputs_that_need_gradients(dm._import((q, k, v)))
    assert {"in_proj_weight", "out_proj.weight"} <= set(need) and len(need) == 5, need


def test_slices_of_run_time_data_become_views():
    """Bounds as the ONNX specification clamps them, negative indices, several axes, steps."""
    from daceml_amd.torch import DaceModule

    class Net(torch.nn.Module):
        def forward(self, x):
            return x[1:, :, -3:] * 2.0, x[:, 0:4:2, :100] + 1.0

    x = torch.randn(3, 5, 7)
    model = DaceModule(Net(), auto_optimize=False)._import((x, ))
    views = {tuple(d.shape): d for d in model.sdfg.arrays.values() if d.view_of is not None}
    a, b = views[(2, 5, 3)], views[(3, 2, 7)]
    assert (a.view_offset, tuple(a.strides)) == (35 + 4, (35, 7, 1))
    assert (b.view_offset, tuple(b.strides)) == (0, (35, 14, 1))
    assert not any(n.schema.name == "Slice" for n in model.sdfg.states()[0].library_nodes())


def test_gradient_through_a_part_that_is_not_a_unit_step_rectangle_is_refused():
    from daceml_amd import graphs
    from daceml_amd.autodiff import AutoDiffException, add_backward_pass
    g = graphs.GraphBuilder("strided_part", torch.float32)
    g.input("x", (4, 6))
    part, _ = g.sdfg.add_view("x_even_rows", "x", (2, 6), (12, 1), 0, find_new_name=False)
    g.output(g.node("Relu", {"X": part}, {"Y": (2, 6)}, label="relu")["Y"], "y")
    with pytest.raises(AutoDiffException, match="rectangular"):
        add_backward_pass(g.sdfg, g.state, ["y"], ["x"])


def _gpu_case():
    torch.manual_seed(3)
    b, heads, p, s = 2, 16, 64, 512      # the shapes of the reference's test
    n = heads * p
    q, k, v = (torch.randn(s, b, n) for _ in range(3))
    return torch.nn.MultiheadAttention(n, heads, bias=False), (q, k, v)


@pytest.mark.gpu
def test_multihead_attention_forward_on_gpu():
    from daceml_amd.torch import DaceModule
    pt, tensors = _gpu_case()
    want, _ = _reference(pt, tensors)
    outs = DaceModule(pt.cuda())(*[t.cuda() for t in tensors])
    for i, (o, w) in enumerate(zip(outs, want)):
        assert_close(o.cpu().numpy(), w, torch.float32, "output %d" % i, rtol=1e-4, atol=2e-5)


@pytest.mark.gpu
def test_multihead_attention_training_on_gpu():
    from daceml_amd.torch import DaceModule
    pt, tensors = _gpu_case()
    r = np.random.default_rng(4)
    dm = DaceModule(pt.cuda(), backward=True)
    ins = [t.cuda().requires_grad_(True) for t in tensors]
    outs = dm(*ins)
    grads = [r.standard_normal(tuple(o.shape)).astype(np.float32) for o in outs]
    torch.autograd.backward(list(outs), [torch.from_numpy(g).cuda() for g in grads])
    _, want = _reference(pt.cpu(), tensors, grads)
    got = [t.grad for t in ins] + [p.grad for p in dm.model.parameters()]
    for i, (g, w) in enumerate(zip(got, want)):
        assert_close(g.cpu().numpy(), w, torch.float32, "gradient %d" % i, rtol=1e-4,
                     atol=2e-5 * max(1.0, float(np.abs(w).max())))
