"""The PyTorch-facing side of the path: ONNX wire reader, importer, DaceModule (cf. the reference's
tests/pytorch/test_module_api.py, tests/pytorch/test_bert_encoder.py, tests/test_models/test_efficientnet.py:
wrap a torch module, call it, compare with the module itself)."""
import collections
import copy
import struct
import warnings

import numpy as np
import pytest
import torch
from torch import nn

from daceml_amd.onnx import proto
from daceml_amd.onnx.onnx_importer import ONNXModel, UnsupportedModel, clean_onnx_name
from daceml_amd.torch import DaceModule, dace_module
from daceml_amd.torch.export import export_onnx
from util import assert_close, host


# ----------------------------------------------------------------------------- modules under test
class SmallEncoder(nn.Module):
    """Linear + GELU + LayerNorm + a 4-head attention with head size 4 + Linear + residual."""
    def __init__(self):
        super().__init__()
        self.l1 = nn.Linear(8, 16)
        self.ln = nn.LayerNorm(16)
        self.l2 = nn.Linear(16, 8)

    def forward(self, x):
        h = self.ln(nn.functional.gelu(self.l1(x)))
        b, t, _ = h.shape
        h = h.view(b, t, 4, 4).permute(0, 2, 1, 3)
        a = torch.softmax(torch.matmul(h, h.transpose(-1, -2)) / 2.0, dim=-1)
        h = torch.matmul(a, h).permute(0, 2, 1, 3).contiguous().view(b, t, 16)
        return self.l2(h) + x


class MBConv(nn.Module):
    """EfficientNet-style block with folded BatchNorm: 1x1 expand, depthwise 3x3 stride 2, squeeze-excite, 1x1 project
    (swish written as x * sigmoid(x), as efficientnet_pytorch's MemoryEfficientSwish exports)."""
    def __init__(self, cin=8, mid=32, cout=16, se=4):
        super().__init__()
        self.expand = nn.Conv2d(cin, mid, 1)
        self.dw = nn.Conv2d(mid, mid, 3, stride=2, padding=1, groups=mid)
        self.se1 = nn.Conv2d(mid, se, 1)
        self.se2 = nn.Conv2d(se, mid, 1)
        self.proj = nn.Conv2d(mid, cout, 1)

    def forward(self, x):
        x = self.expand(x)
        x = x * torch.sigmoid(x)
        x = self.dw(x)
        x = x * torch.sigmoid(x)
        s = nn.functional.adaptive_avg_pool2d(x, 1)
        s = self.se1(s)
        s = s * torch.sigmoid(s)
        s = self.se2(s)
        x = torch.sigmoid(s) * x
        return self.proj(x)


class BertLayerOutput(nn.Module):
    """HuggingFace BertLayer (what tests/pytorch/test_bert_encoder.py wraps), returning the hidden states only."""
    def __init__(self, hidden, heads, ffn):
        super().__init__()
        from transformers import BertConfig
        from transformers.models.bert.modeling_bert import BertLayer
        cfg = BertConfig(hidden_size=hidden, num_attention_heads=heads, intermediate_size=ffn,
                         hidden_dropout_prob=0.0, attention_probs_dropout_prob=0.0)
        cfg._attn_implementation = "eager"
        self.layer = BertLayer(cfg)

    def forward(self, x):
        out = self.layer(x)
        return out[0] if isinstance(out, (tuple, list)) else out


class ConvBN(nn.Module):
    """Conv -> BatchNorm -> ReLU -> Conv, the un-folded form of an EfficientNet stem."""
    def __init__(self, track=True):
        super().__init__()
        self.conv = nn.Conv2d(3, 8, 3, padding=1)
        self.bn = nn.BatchNorm2d(8, track_running_stats=track)
        self.out = nn.Conv2d(8, 4, 1)

    def forward(self, x):
        return self.out(torch.relu(self.bn(self.conv(x))))


def _kinds(sdfg):
    return collections.Counter(n.schema.name for st in sdfg.states() for n in st.library_nodes())


# ----------------------------------------------------------------------------- wire reader
def _varint(v):
    v &= (1 << 64) - 1
    out = bytearray()
    while True:
        b = v & 0x7F
        v >>= 7
        out.append(b | (0x80 if v else 0))
        if not v:
            return bytes(out)


def _ld(num, payload):
    return _varint(num << 3 | 2) + _varint(len(payload)) + payload


def test_wire_reader_decodes_hand_built_messages():
    # a TensorProto with dims [2, 2], int64 data given unpacked (one of them negative) and a name
    t = _ld(1, _varint(2) + _varint(2)) + _varint(2 << 3) + _varint(7) + b"".join(
        _varint(7 << 3) + _varint(v) for v in (1, -2, 3, 1 << 40)) + _ld(8, b"t0")
    tp = proto.TensorProto(t)
    assert tp.name == "t0" and tp.array.dtype == np.int64 and tp.array.tolist() == [[1, -2], [3, 1 << 40]]
    # fp16 values travel as bit patterns in int32_data (packed here)
    bits = np.array([1.5, -0.25], np.float16).view(np.uint16).tolist()
    t = _ld(1, _varint(2)) + _varint(2 << 3) + _varint(10) + _ld(5, b"".join(_varint(b) for b in bits))
    assert proto.TensorProto(t).array.tolist() == [1.5, -0.25]
    # raw_data, float
    t = _ld(1, _varint(3)) + _varint(2 << 3) + _varint(1) + _ld(9, struct.pack("<3f", 1.0, 2.0, -3.5))
    assert proto.TensorProto(t).array.tolist() == [1.0, 2.0, -3.5]
    # attributes: INT (negative), FLOAT, INTS packed, STRING
    a = proto.AttributeProto(_ld(1, b"axis") + _varint(3 << 3) + _varint(-1) + _varint(20 << 3) + _varint(2))
    assert (a.name, a.value) == ("axis", -1)
    a = proto.AttributeProto(_ld(1, b"alpha") + _varint(2 << 3 | 5) + struct.pack("<f", 0.5) + _varint(20 << 3) + _varint(1))
    assert a.value == 0.5
    a = proto.AttributeProto(_ld(1, b"perm") + _ld(8, _varint(0) + _varint(2) + _varint(1)) + _varint(20 << 3) + _varint(7))
    assert a.value == [0, 2, 1]
    a = proto.AttributeProto(_ld(1, b"auto_pad") + _ld(4, b"NOTSET") + _varint(20 << 3) + _varint(3))
    assert a.value == "NOTSET"
    with pytest.raises(proto.ProtoError):
        proto.TensorProto(t[:-3])                      # truncated
    with pytest.raises(proto.ProtoError):
        proto.load_model(_varint(1 << 3) + _varint(7))   # no graph


def test_wire_reader_on_an_exported_model():
    m = nn.Sequential(nn.Linear(8, 16), nn.GELU(), nn.LayerNorm(16))
    model = proto.load_model(export_onnx(m, (torch.randn(2, 4, 8), )))
    assert model.opset_import[""] == 12 and model.producer_name == "pytorch"
    g = model.graph
    ops = [n.op_type for n in g.node if n.op_type != "Constant"]
    # nn.Linear = Transpose, MatMul, Add; exact GELU = Div, Erf, Add, Mul, Mul; LayerNorm = the nine-node chain
    assert ops == ["Transpose", "MatMul", "Add", "Div", "Erf", "Add", "Mul", "Mul", "ReduceMean", "Sub", "Pow",
                   "ReduceMean", "Add", "Sqrt", "Div", "Mul", "Add"]
    inits = {t.name: t.array for t in g.initializer}
    sd = m.state_dict()
    assert set(inits) == set(sd)
    for k, v in sd.items():
        assert np.array_equal(inits[k], v.numpy())
    x = [i for i in g.input if i.name not in inits]
    assert len(x) == 1 and x[0].shape == [2, 4, 8] and x[0].elem_type == 1
    consts = [n.attribute[0].value for n in g.node if n.op_type == "Constant"]
    assert [round(float(c), 5) for c in consts] == [1.41421, 1.0, 0.5, 2.0, 1e-05]


# ----------------------------------------------------------------------------- importer
def test_importer_names_shapes_and_folding():
    net = SmallEncoder()
    model = ONNXModel("enc", export_onnx(net, (torch.randn(2, 4, 8), )), auto_optimize=False)
    sdfg = model.sdfg
    assert model.outputs == ["__return"] and len(model.inputs) == 1
    assert set(model.weights) == set(net.state_dict())
    assert clean_onnx_name("l1.weight") == "l1DOTweight" and clean_onnx_name("0.bias") == "ONNX_0DOTbias"
    assert sdfg.arrays["l1DOTweight"].shape == (16, 8) and not sdfg.arrays["l1DOTweight"].transient
    assert sdfg.arrays["__return"].shape == (2, 4, 8)
    kinds = _kinds(sdfg)
    # the Shape / Gather / Unsqueeze / Concat chains around view() are evaluated at import
    assert not {"Shape", "Gather", "Unsqueeze", "Concat", "Constant"} & set(kinds)
    assert kinds["Reshape"] == 2 and kinds["Softmax"] == 1 and kinds["MatMul"] == 4 and kinds["Transpose"] == 5
    reshapes = [n for n in model.state.library_nodes() if n.schema.name == "Reshape"]
    shapes = sorted(sdfg.arrays[e.data.data].shape for r in reshapes for e in model.state.out_edges(r))
    assert shapes == [(2, 4, 4, 4), (2, 4, 16)]
    stats = model.auto_optimize()
    assert stats["gelu"] == 1 and stats["layernorm"] == 1 and stats["matmul_to_einsum"] == 4
    assert _kinds(sdfg) == {"FusedEinsum": 3, "Einsum": 1, "Softmax": 1, "Gelu": 1, "LayerNormalization": 1}


def test_importer_refuses_what_it_cannot_run():
    class Odd(nn.Module):
        def forward(self, x):
            return torch.cumsum(x, dim=1)

    with pytest.raises(UnsupportedModel, match="Unsupported ONNX operator: 'CumSum'"):
        ONNXModel("odd", export_onnx(Odd(), (torch.randn(2, 3), )))


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
def test_huggingface_bert_layer_imports_to_the_fused_graph(dtype):
    """The decomposition the real exporter emits for BertLayer is the one the hand-built bench graph assumes: after
    the fusion pipeline both consist of the same library nodes."""
    from daceml_amd import graphs
    from daceml_amd.transformation import fusion
    b, s, h, heads, ffn = 2, 64, 256, 4, 512
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        m = DaceModule(BertLayerOutput(h, heads, ffn).eval().to(dtype), backward=True)
        model = m._import((torch.randn(b, s, h).to(dtype), ))
    want = graphs.bert_encoder_layer(b, s, h, heads, ffn, dtype, eps=1e-12)
    want_stats = fusion.auto_optimize(want, training=True)
    assert _kinds(model.sdfg) == _kinds(want)
    for k in ("gelu", "layernorm", "attention", "epilogues", "skip_layernorm"):
        assert m.optimization_stats[k] == want_stats[k], k
    if dtype == torch.float16:
        assert _kinds(model.sdfg)["FusedAttention"] == 1
    # parameters are graph inputs under their state_dict names
    assert "layer.attention.self.query.weight" in model.inputs and not model.weights


def test_batchnorm_import_forms():
    """eval -> inference form (Y only); training -> all five outputs, with the running statistics as graph inputs
    under their buffer names (so that the node's write-back updates the module's buffers)."""
    x = torch.randn(2, 3, 8, 8)
    m = DaceModule(ConvBN().eval(), auto_optimize=False)
    model = m._import((x, ))
    bn = [n for n in model.state.library_nodes() if n.schema.name == "BatchNormalization"]
    assert len(bn) == 1 and {e.src_conn for e in model.state.out_edges(bn[0])} == {"Y"}
    assert {e.dst_conn for e in model.state.in_edges(bn[0])} == {"X", "scale", "B", "in_mean", "in_var"}
    assert abs(bn[0].momentum - 0.9) < 1e-6 and abs(bn[0].epsilon - 1e-5) < 1e-9
    m = DaceModule(ConvBN().train(), training=True, backward=True, auto_optimize=False)
    model = m._import((x, ))
    bn = [n for n in model.state.library_nodes() if n.schema.name == "BatchNormalization"]
    assert {e.src_conn for e in model.state.out_edges(bn[0])} == {"Y", "out_mean", "out_var", "saved_mean", "saved_var"}
    assert "bn.running_mean" in model.inputs and "bn.running_var" in model.inputs
    assert model.sdfg.arrays["SLASHbnSLASHBatchNormalization_output_3"].shape == (8, )


def test_module_hooks_and_decorator():
    calls = []
    m = DaceModule(SmallEncoder(), auto_optimize=False)
    m.append_post_onnx_hook("b", lambda mod: calls.append("b"))
    m.prepend_post_onnx_hook("a", lambda mod: calls.append("a"))
    m.append_post_onnx_hook("b", lambda mod: calls.append("b2"))       # same name: made unique, both run
    assert list(m.post_onnx_hooks) == ["a", "b", "b_0"]
    m._import((torch.randn(2, 4, 8), ))
    assert calls == ["a", "b", "b2"]
    assert _kinds(m.sdfg)["MatMul"] == 4                                # nothing was fused
    auto = DaceModule(SmallEncoder(), backward=True)
    assert list(auto.post_onnx_hooks) == ["auto_optimize"] and list(auto.post_autodiff_hooks) == ["auto_optimize"]
    with pytest.raises(ValueError):
        DaceModule(SmallEncoder(), cuda=False)

    @dace_module(backward=True)
    class Wrapped(nn.Module):
        def __init__(self, n):
            super().__init__()
            self.fc = nn.Linear(n, n)

        def forward(self, x):
            return self.fc(x)

    w = Wrapped(4)
    assert isinstance(w, DaceModule) and isinstance(w.model.fc, nn.Linear) and w.backward


# ----------------------------------------------------------------------------- on the GPU
def _compare_module(module, x, dtype, backward, rtol=None, atol=None, grad_rtol=None, grad_atol=None):
    module = module.cuda().to(dtype)
    ref = copy.deepcopy(module).double()
    x = x.cuda().to(dtype)
    wrapped = DaceModule(module, backward=backward)
    xr = x.detach().double().requires_grad_(backward)
    xs = x.detach().clone().requires_grad_(backward)
    y = wrapped(xs)
    want = ref(xr)
    assert y.dtype == dtype and y.shape == want.shape
    assert_close(host(y), want.detach().cpu().numpy(), dtype, "forward", rtol=rtol, atol=atol)
    if not backward:
        return wrapped
    g = torch.randn(want.shape, generator=torch.Generator().manual_seed(5)).cuda()
    y.backward(g.to(dtype))
    want.backward(g.to(dtype).double())
    assert_close(host(xs.grad), xr.grad.cpu().numpy(), dtype, "input gradient", rtol=grad_rtol, atol=grad_atol)
    for (n, p), (_, pr) in zip(module.named_parameters(), ref.named_parameters()):
        assert p.grad is not None, n
        scale = float(pr.grad.abs().max())
        a = (grad_atol if grad_atol is not None else (1e-2 if dtype == torch.float16 else 1e-6))
        assert_close(host(p.grad), pr.grad.cpu().numpy(), dtype, "gradient of " + n, rtol=grad_rtol,
                     atol=a * max(scale, 1.0))
    return wrapped


@pytest.mark.gpu
@pytest.mark.parametrize("backward", [False, True])
def test_small_encoder_module(backward):
    torch.manual_seed(0)
    # a chain of seven fp32 nodes: rounding accumulates beyond one node's 1e-5 / 1e-6
    w = _compare_module(SmallEncoder(), torch.randn(2, 4, 8), torch.float32, backward, rtol=1e-4, atol=1e-5,
                        grad_rtol=1e-4, grad_atol=1e-5)
    assert w.optimization_stats["gelu"] == 1 and w.optimization_stats["layernorm"] == 1
    # a second call reuses the bound program and sees updated parameters
    with torch.no_grad():
        w.model.l2.bias.add_(1.0)
    x = torch.randn(2, 4, 8, device="cuda")
    assert_close(host(w(x)), host(w.model(x)), torch.float32, "second call", rtol=1e-4, atol=1e-5)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,backward", [(torch.float32, False), (torch.float16, False), (torch.float16, True)])
def test_huggingface_bert_layer_module(dtype, backward):
    torch.manual_seed(1)
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        layer = BertLayerOutput(256, 4, 512).eval()
        kw = dict(rtol=1e-4, atol=2e-5) if dtype == torch.float32 else {}
        w = _compare_module(layer, torch.randn(2, 128, 256), dtype, backward, **kw)
    kinds = {l.kind for l in w.compiled.launches}
    if dtype == torch.float16:
        assert "attention" in kinds and w.optimization_stats["attention"] == 1
        if backward:
            assert "attention_backward" in kinds and w.optimization_stats["grouped_einsums"] > 0


@pytest.mark.gpu
def test_mbconv_module():
    torch.manual_seed(2)
    w = _compare_module(MBConv(), torch.randn(3, 8, 32, 32), torch.float32, False, rtol=1e-4, atol=1e-5)
    assert w.optimization_stats["swish"] == 3 and w.optimization_stats["gated_conv"] == 1


@pytest.mark.gpu
def test_onnx_model_call_passes_its_own_weights():
    """ONNXModel on its own (daceml/onnx/onnx_importer.py:482-560): initializers become ``weights`` that every call
    passes; inputs positionally or by name."""
    torch.manual_seed(3)
    net = SmallEncoder()
    model = ONNXModel("enc", export_onnx(net, (torch.randn(2, 4, 8), )))
    x = torch.randn(2, 4, 8)
    want = net(x).detach().numpy()
    assert_close(host(model(x.cuda())), want, torch.float32, "positional", rtol=1e-4, atol=1e-5)
    assert_close(host(model(**{model.inputs[0]: x.cuda()})), want, torch.float32, "by name", rtol=1e-4, atol=1e-5)
    with pytest.raises(TypeError):
        model()


@pytest.mark.gpu
def test_batchnorm_module_training_and_eval():
    """nn.BatchNorm2d inside a module (the reference's test_bn_in_import, tests/test_shared_input_output.py:46-68,
    plus the backward pass and the running statistics)."""
    torch.manual_seed(4)
    net = ConvBN().cuda().train()
    ref = copy.deepcopy(net).double()
    w = DaceModule(net, training=True, backward=True)
    x = torch.randn(6, 3, 16, 16, device="cuda")
    xs = x.clone().requires_grad_(True)
    xr = x.double().requires_grad_(True)
    y, want = w(xs), ref(xr)
    assert_close(host(y), want.detach().cpu().numpy(), torch.float32, "training forward", rtol=1e-4, atol=1e-5)
    g = torch.randn_like(y)
    y.backward(g)
    want.backward(g.double())
    assert_close(host(xs.grad), xr.grad.cpu().numpy(), torch.float32, "dx", rtol=1e-4, atol=1e-5)
    for (n, p), (_, pr) in zip(net.named_parameters(), ref.named_parameters()):
        scale = max(float(pr.grad.abs().max()), 1.0)
        assert_close(host(p.grad), pr.grad.cpu().numpy(), torch.float32, "gradient of " + n, rtol=1e-4, atol=1e-5 * scale)
    # running statistics were updated in the module's own buffers: the mean as torch does, the variance with the
    # biased batch variance (the reference's rule) where torch uses the unbiased one
    assert_close(host(net.bn.running_mean), ref.bn.running_mean.cpu().numpy(), torch.float32, "running mean",
                 rtol=1e-4, atol=1e-6)
    cnt = 6 * 16 * 16
    unbiased = (ref.bn.running_var.cpu().numpy() - 0.9) / 0.1
    assert_close(host(net.bn.running_var), 0.9 + 0.1 * unbiased * (cnt - 1) / cnt, torch.float32, "running var",
                 rtol=1e-4, atol=1e-6)
    # evaluation mode: the inference form with those statistics
    net_eval = copy.deepcopy(net).eval()
    we = DaceModule(copy.deepcopy(net_eval))
    assert_close(host(we(x)), host(net_eval(x)), torch.float32, "eval forward", rtol=1e-4, atol=1e-5)


class TwoInTwoOut(nn.Module):
    def __init__(self):
        super().__init__()
        self.fc = nn.Linear(16, 16)

    def forward(self, a, b):
        h = self.fc(a) * torch.sigmoid(b)
        return h + a, torch.tanh(h)


@pytest.mark.gpu
def test_module_with_two_inputs_two_outputs_and_a_skipped_gradient():
    """Several inputs and outputs, one input excluded from differentiation (`inputs_to_skip`,
    daceml/torch/module.py:59-60): its gradient comes back as None, everything else matches autograd."""
    torch.manual_seed(6)
    net = TwoInTwoOut().cuda()
    ref = copy.deepcopy(net).double()
    probe = DaceModule(copy.deepcopy(net))
    model = probe._import((torch.randn(4, 16, device="cuda"), torch.randn(4, 16, device="cuda")))
    assert len(model.inputs) == 2 + 2 and model.outputs == ["__return_0", "__return_1"]
    skip = model.inputs[1]
    w = DaceModule(net, backward=True, inputs_to_skip=[skip])
    a = torch.randn(4, 16, device="cuda", requires_grad=True)
    b = torch.randn(4, 16, device="cuda", requires_grad=True)
    ar, br = a.detach().double().requires_grad_(True), b.detach().double().requires_grad_(True)
    y0, y1 = w(a, b)
    r0, r1 = ref(ar, br)
    assert_close(host(y0), r0.detach().cpu().numpy(), torch.float32, "first output", rtol=1e-4, atol=1e-5)
    assert_close(host(y1), r1.detach().cpu().numpy(), torch.float32, "second output", rtol=1e-4, atol=1e-5)
    g0, g1 = torch.randn_like(y0), torch.randn_like(y1)
    torch.autograd.backward([y0, y1], [g0, g1])
    torch.autograd.backward([r0, r1], [g0.double(), g1.double()])
    assert b.grad is None
    assert_close(host(a.grad), ar.grad.cpu().numpy(), torch.float32, "gradient of the first input", rtol=1e-4, atol=1e-5)
    for (n, p_), (_, pr) in zip(net.named_parameters(), ref.named_parameters()):
        assert_close(host(p_.grad), pr.grad.cpu().numpy(), torch.float32, "gradient of " + n, rtol=1e-4, atol=1e-5)
    # only one of the two output gradients given: the other counts as zero
    a2 = a.detach().clone().requires_grad_(True)
    ar2 = a.detach().double().requires_grad_(True)
    w(a2, b.detach())[1].sum().backward()
    ref(ar2, b.detach().double())[1].sum().backward()
    assert_close(host(a2.grad), ar2.grad.cpu().numpy(), torch.float32, "partial output gradient", rtol=1e-4, atol=1e-5)


@pytest.mark.gpu
def test_parameter_to_transient():
    """The reference's own test of this transformation (tests/transformation/test_param_to_transient.py): a Linear
    layer whose weight becomes a buffer of the compiled program. On top of it: the program works on a snapshot (a
    later change of the nn.Parameter is not seen) and the weight is no longer an argument."""
    from daceml_amd.transformation import parameter_to_transient

    class Module(nn.Module):
        def __init__(self):
            super().__init__()
            self.fc1 = nn.Linear(10, 3)

        def forward(self, x):
            return self.fc1(x)

    torch.manual_seed(3)
    pt_module = Module().cuda()
    dace_module = Module().cuda()
    dace_module.load_state_dict(pt_module.state_dict())
    x = torch.rand(2, 10).cuda()
    plain = DaceModule(dace_module)
    assert torch.allclose(plain(x), pt_module(x), rtol=1e-5, atol=1e-6)
    assert "fc1DOTweight" in plain.compiled.arglist()

    wrapped = DaceModule(dace_module)
    wrapped.append_post_onnx_hook("param_to_transient", lambda model: parameter_to_transient(model, "fc1.weight"))
    want = pt_module(x)
    assert torch.allclose(wrapped(x), want, rtol=1e-5, atol=1e-6)
    assert "fc1DOTweight" not in wrapped.compiled.arglist() and "fc1.weight" not in wrapped.dace_model.inputs
    assert "init_fc1.weight" in wrapped.post_compile_hooks
    with torch.no_grad():
        dace_module.fc1.weight.mul_(2.0)          # the snapshot does not follow the parameter ...
        dace_module.fc1.bias.add_(1.0)            # ... an ordinary parameter does
    assert torch.allclose(wrapped(x), want + 1.0, rtol=1e-5, atol=1e-6)
    with pytest.raises(ValueError):
        again = DaceModule(dace_module)
        again.append_post_onnx_hook("twice", lambda model: (parameter_to_transient(model, "fc1.weight"),
                                                           parameter_to_transient(model, "fc1.weight")))
        again(x)


class MBConvBN(nn.Module):
    """MBConv block as efficientnet_pytorch builds it (what tests/autodiff/torch/test_efficientnet_block_backward.py
    trains): every conv without bias followed by BatchNorm, swish as x * sigmoid(x), squeeze-excite with biases."""
    def __init__(self, cin=8, mid=32, cout=16, se=4):
        super().__init__()
        self.expand, self.bn0 = nn.Conv2d(cin, mid, 1, bias=False), nn.BatchNorm2d(mid)
        self.dw, self.bn1 = nn.Conv2d(mid, mid, 3, stride=1, padding=1, groups=mid, bias=False), nn.BatchNorm2d(mid)
        self.se1, self.se2 = nn.Conv2d(mid, se, 1), nn.Conv2d(se, mid, 1)
        self.proj, self.bn2 = nn.Conv2d(mid, cout, 1, bias=False), nn.BatchNorm2d(cout)

    def forward(self, x):
        x = self.bn0(self.expand(x))
        x = x * torch.sigmoid(x)
        x = self.bn1(self.dw(x))
        x = x * torch.sigmoid(x)
        s = nn.functional.adaptive_avg_pool2d(x, 1)
        s = self.se1(s)
        s = s * torch.sigmoid(s)
        s = self.se2(s)
        x = torch.sigmoid(s) * x
        return self.bn2(self.proj(x))


@pytest.mark.gpu
def test_mbconv_block_training_through_the_wrapper():
    torch.manual_seed(7)
    net = MBConvBN().cuda().train()
    ref = copy.deepcopy(net).double()
    w = DaceModule(net, training=True, backward=True)
    x = torch.randn(4, 8, 12, 12, device="cuda")
    xs, xr = x.clone().requires_grad_(True), x.double().requires_grad_(True)
    y, want = w(xs), ref(xr)
    assert_close(host(y), want.detach().cpu().numpy(), torch.float32, "forward", rtol=2e-4, atol=2e-5)
    g = torch.randn_like(y)
    y.backward(g)
    want.backward(g.double())
    kinds = {l.kind for l in w.compiled.launches}
    assert {"batchnorm", "batchnorm_backward", "conv"} <= kinds
    assert_close(host(xs.grad), xr.grad.cpu().numpy(), torch.float32, "dx", rtol=1e-3, atol=1e-4)
    for (n, p_), (_, pr) in zip(net.named_parameters(), ref.named_parameters()):
        scale = max(float(pr.grad.abs().max()), 1.0)
        assert_close(host(p_.grad), pr.grad.cpu().numpy(), torch.float32, "gradient of " + n, rtol=1e-3, atol=1e-4 * scale)


# ----------------------------------------------------------------------------- what a pending backward depends on
def _small_encoder_reference(net, x64, gy64):
    ref = copy.deepcopy(net).double()
    xr = x64.clone().requires_grad_(True)
    ref(xr).backward(gy64)
    return xr.grad, {n: p_.grad for n, p_ in ref.named_parameters()}


@pytest.mark.gpu
def test_backward_survives_dropped_and_overwritten_inputs():
    """The dispatcher saves what backward reads on the autograd context (daceml/torch/dispatchers/ctypes_module.py:
    150-170): a non-contiguous input (whose dense copy nobody else owns) and an input that the caller drops and
    whose memory is reused before ``backward()`` still give autograd's gradients."""
    torch.manual_seed(11)
    net = SmallEncoder().cuda()
    w = DaceModule(copy.deepcopy(net), backward=True)
    base = torch.randn(8, 3, 5, device="cuda")           # [feature, batch, time]: the permuted view is not dense
    gy = torch.randn(3, 5, 8, device="cuda")
    want_dx, want = _small_encoder_reference(net, base.permute(1, 2, 0).double(), gy.double())

    leaf = base.clone().requires_grad_(True)
    x = leaf.permute(1, 2, 0)
    assert not x.is_contiguous()
    y = w(x)
    del x
    # churn the caching allocator: same-sized blocks are handed out again and overwritten
    junk = [torch.full((3, 5, 8), float("nan"), device="cuda") for _ in range(64)]
    junk += [torch.full((3, 5, 16), float("nan"), device="cuda") for _ in range(64)]
    y.backward(gy)
    del junk
    assert_close(host(leaf.grad.permute(1, 2, 0)), want_dx.cpu().numpy(), torch.float32, "dx", rtol=1e-4, atol=1e-5)
    for n, p_ in w.model.named_parameters():
        assert_close(host(p_.grad), want[n].cpu().numpy(), torch.float32, "gradient of " + n, rtol=1e-4, atol=1e-5)

    # an activation of an upstream layer that only the graph owns: w(embedding(ids))
    w2 = DaceModule(copy.deepcopy(net), backward=True)
    emb = nn.Embedding(10, 8).cuda()
    ids = torch.randint(0, 10, (3, 5), device="cuda")
    y = w2(emb(ids))
    junk = [torch.full((3, 5, 8), float("nan"), device="cuda") for _ in range(64)]
    y.backward(gy)
    del junk
    _, want2 = _small_encoder_reference(net, emb(ids).detach().double(), gy.double())
    for n, p_ in w2.model.named_parameters():
        assert_close(host(p_.grad), want2[n].cpu().numpy(), torch.float32, "gradient of " + n + " (embedding input)",
                     rtol=1e-4, atol=1e-5)


@pytest.mark.gpu
def test_two_forward_calls_pending_before_their_backward_calls():
    """Each forward call keeps its own copies of the buffers its backward call reads, so backward calls may come
    in any order after several forward calls (as with the reference's dispatcher)."""
    torch.manual_seed(12)
    net = SmallEncoder().cuda()
    w = DaceModule(copy.deepcopy(net), backward=True)
    assert w.function is None
    xs = [torch.randn(3, 5, 8, device="cuda", requires_grad=True) for _ in range(2)]
    gys = [torch.randn(3, 5, 8, device="cuda") for _ in range(2)]
    ys = [w(x) for x in xs]
    assert w.forwarded_transients, "the backward state reads buffers the forward state fills"
    for i in (0, 1):                                    # first call's backward after the second call's forward
        ys[i].backward(gys[i])
    total = {n: torch.zeros_like(p_, dtype=torch.float64) for n, p_ in net.named_parameters()}
    for i in (0, 1):
        dx, grads = _small_encoder_reference(net, xs[i].detach().double(), gys[i].double())
        assert_close(host(xs[i].grad), dx.cpu().numpy(), torch.float32, "dx of call %d" % i, rtol=1e-4, atol=1e-5)
        for n in total:
            total[n] += grads[n]
    for n, p_ in w.model.named_parameters():
        assert_close(host(p_.grad), total[n].cpu().numpy(), torch.float32, "accumulated gradient of " + n,
                     rtol=1e-4, atol=2e-5)


class HiddenAndPooled(nn.Module):
    def __init__(self):
        super().__init__()
        self.fc = nn.Linear(16, 16)

    def forward(self, a):
        h = torch.sigmoid(self.fc(a))
        return h, torch.tanh(h)


@pytest.mark.gpu
def test_module_returning_an_intermediate_and_a_function_of_it():
    """An output that another node of the graph also reads receives the caller's gradient PLUS the consumer's."""
    torch.manual_seed(13)
    net = HiddenAndPooled().cuda()
    ref = copy.deepcopy(net).double()
    w = DaceModule(net, backward=True)
    a = torch.randn(4, 16, device="cuda", requires_grad=True)
    ar = a.detach().double().requires_grad_(True)
    h, t = w(a)
    hr, tr = ref(ar)
    g0, g1 = torch.randn_like(h), torch.randn_like(t)
    keep0 = g0.clone()
    torch.autograd.backward([h, t], [g0, g1])
    torch.autograd.backward([hr, tr], [g0.double(), g1.double()])
    assert torch.equal(g0, keep0), "the caller's gradient buffer is read only"
    assert_close(host(a.grad), ar.grad.cpu().numpy(), torch.float32, "gradient of the input", rtol=1e-4, atol=1e-5)
    for (n, p_), (_, pr) in zip(net.named_parameters(), ref.named_parameters()):
        assert_close(host(p_.grad), pr.grad.cpu().numpy(), torch.float32, "gradient of " + n, rtol=1e-4, atol=1e-5)
