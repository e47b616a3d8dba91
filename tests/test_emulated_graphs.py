"""Whole graphs without a GPU: the BERT encoder layer - as the exporter emits it, and after the fusion passes - is
differentiated, expanded, and the calls its tasklets make are interpreted by tests/abi_emulator.py on NumPy arrays.
Compared with the oracle, this checks everything on the host side of the C ABI for the headline workload: the fusion
passes, the reverse nodes and gradient accumulation of the autodiff generator, the views that replace Transpose /
Reshape nodes, every descriptor, operand order, pointer table and workspace offset. (The kernels behind the ABI are
checked against the same oracle in tests/test_gpu_graphs.py.)"""
import numpy as np
import pytest
import torch

from oracle import bert_layer as OB
from tests.abi_emulator import run_sdfg
from tests.util import assert_close, rng

B, S, H, HEADS, FFN = 2, 64, 128, 2, 256


def _inputs(dtype, seed=1234):
    npdt = np.float16 if dtype == torch.float16 else np.float32
    p = OB.init_params(H, FFN, seed, np.float32, bias_std=0.02)
    r = rng(seed + 1)
    p["ln1_g"], p["ln2_g"] = r.uniform(0.5, 1.5, H).astype(np.float32), r.uniform(0.5, 1.5, H).astype(np.float32)
    p["ln1_b"], p["ln2_b"] = (r.standard_normal(H) * 0.1).astype(np.float32), (r.standard_normal(H) * 0.1).astype(np.float32)
    x = r.standard_normal((B, S, H)).astype(npdt)
    dy = rng(77).standard_normal((B, S, H)).astype(npdt)
    return x, dy, {k: v.astype(npdt) for k, v in p.items()}


def _oracle(x, dy, p):
    x64, p64 = x.astype(np.float64), {k: v.astype(np.float64) for k, v in p.items()}
    y, saved = OB.forward(x64, p64, HEADS, eps=1e-5, keep=True)
    return y, OB.backward(x64, p64, HEADS, dy.astype(np.float64), saved, eps=1e-5, term_scales=True)


def _check(arrays, x, dy, p, dtype, grads=True):
    y, want = _oracle(x, dy, p)
    f16 = dtype == torch.float16
    assert_close(arrays["y"], y, dtype, "y", **({} if f16 else dict(rtol=1e-4, atol=2e-5)))
    if not grads:
        return
    assert_close(arrays["gradient_x"], want["x"], dtype, "dx", **({} if f16 else dict(rtol=1e-4, atol=2e-5)))
    for n in OB.PARAM_NAMES:
        scale = float(np.abs(want[n]).max())
        # fp16: on top of the stated tolerance, what a sum over the rows of products of fp16-stored tensors can be off by
        tol = dict(rtol=2e-2, atol=1e-2 + 16.0 * 2.0 ** -11 * want["terms:" + n]) if f16 \
            else dict(rtol=1e-4, atol=1e-5 * max(scale, 1.0))
        assert_close(arrays["gradient_" + n], want[n], dtype, "d" + n, **tol)


@pytest.mark.parametrize("dtype,attention", [(torch.float16, True), (torch.float16, False), (torch.float32, False)])
def test_fused_bert_layer_forward_and_backward(dtype, attention):
    from daceml_amd import graphs
    from daceml_amd.autodiff import add_backward_pass
    from daceml_amd.runtime import expand_onnx_nodes
    from daceml_amd.transformation import fusion
    x, dy, p = _inputs(dtype)
    sdfg = graphs.bert_encoder_layer(B, S, H, HEADS, FFN, dtype, eps=1e-5)
    fusion.auto_optimize(sdfg, training=True, attention=attention, gelu_epilogue=not attention)
    add_backward_pass(sdfg, sdfg.states()[0], ["y"], ["x"] + OB.PARAM_NAMES,
                      grad_dtypes={n: torch.float32 for n in OB.PARAM_NAMES})
    if attention:
        fusion.optimize_backward(sdfg)
    expand_onnx_nodes(sdfg)
    arrays = {"x": x.copy(), "gradient_y": dy.copy(), **{k: v.copy() for k, v in p.items()}}
    log = run_sdfg(sdfg, arrays)
    if attention:
        assert sorted(set(log)) == ["dmlhip_attention_backward_f16", "dmlhip_attention_f16", "dmlhip_gemm_f16_grouped",
                                    "dmlhip_gemm_f16_grouped_asum", "dmlhip_gemm_f16_ksum", "dmlhip_gemm_f16_ws",
                                    "dmlhip_layernorm_backward_f16", "dmlhip_layernorm_f16", "dmlhip_unary_backward_f16",
                                    "dmlhip_unary_f16"]
        assert len(log) == 19       # the launch count of the benchmarked step
    _check(arrays, x, dy, p, dtype)
    # inputs are read-only
    assert np.array_equal(arrays["x"], x) and all(np.array_equal(arrays[k], v) for k, v in p.items())


def test_exporter_form_bert_layer_differentiates_without_any_fusion():
    """The graph exactly as imported (MatMul, Reshape, Transpose, the nine-node LayerNorm and five-node GELU chains):
    every node has a reverse implementation, among them MatMul (the reference expands it to an Einsum first,
    backward_pass_generator.py:425-494) and Reshape."""
    from daceml_amd import graphs
    from daceml_amd.autodiff import add_backward_pass
    from daceml_amd.runtime import expand_onnx_nodes
    dtype = torch.float32
    x, dy, p = _inputs(dtype)
    sdfg = graphs.bert_encoder_layer(B, S, H, HEADS, FFN, dtype, eps=1e-5)
    names = {n.schema.name for n in sdfg.states()[0].library_nodes()}
    assert {"MatMul", "Reshape", "Transpose", "ReduceMean", "Pow", "Sqrt", "Erf", "Softmax"} <= names
    grads = add_backward_pass(sdfg, sdfg.states()[0], ["y"], ["x"] + OB.PARAM_NAMES)
    assert set(grads) == {"x"} | set(OB.PARAM_NAMES)
    expand_onnx_nodes(sdfg)
    arrays = {"x": x.copy(), "gradient_y": dy.copy(), **{k: v.copy() for k, v in p.items()}}
    run_sdfg(sdfg, arrays)
    _check(arrays, x, dy, p, dtype)


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_inference_graph(dtype):
    from daceml_amd import graphs
    from daceml_amd.runtime import expand_onnx_nodes
    from daceml_amd.transformation import fusion
    x, dy, p = _inputs(dtype)
    sdfg = graphs.bert_encoder_layer(B, S, H, HEADS, FFN, dtype, eps=1e-5)
    fusion.auto_optimize(sdfg)
    expand_onnx_nodes(sdfg)
    arrays = {"x": x.copy(), **{k: v.copy() for k, v in p.items()}}
    run_sdfg(sdfg, arrays)
    _check(arrays, x, dy, p, dtype, grads=False)


def test_masked_attention_graph_forward_and_backward():
    """The chain with the additive mask through fusion, autodiff and the masked entry points."""
    from daceml_amd.autodiff import add_backward_pass
    from daceml_amd.runtime import expand_onnx_nodes
    from daceml_amd.transformation import fusion
    from oracle import ops as O
    from tests.test_zx_attention_mask import _chain
    b, h, sq, sk = 2, 3, 40, 48
    g = _chain((b, 1, 1, sk), b=b, h=h, sq=sq, sk=sk)
    assert fusion.auto_optimize(g.sdfg)["attention"] == 1
    add_backward_pass(g.sdfg, g.state, ["o"], ["q", "k", "v"])
    expand_onnx_nodes(g.sdfg)
    r = rng(5)
    q, k, v = (r.standard_normal((b, h, n, 64)).astype(np.float16) for n in (sq, sk, sk))
    do = r.standard_normal((b, h, sq, 64)).astype(np.float16)
    mask = np.zeros((b, 1, 1, sk), np.float16)
    mask[1, :, :, 30:] = -10000.0
    arrays = {"q": q.copy(), "k": k.copy(), "v": v.copy(), "mask": mask.copy(), "gradient_o": do.copy()}
    log = run_sdfg(g.sdfg, arrays)
    assert log == ["dmlhip_attention_masked_f16", "dmlhip_attention_masked_backward_f16"]
    f64 = lambda t: t.astype(np.float64)  # noqa: E731
    want, _ = O.attention(f64(q), f64(k), f64(v), 0.125, f64(mask))
    assert_close(arrays["o"], want, torch.float16, "masked attention (emulated)")
    for name, w in zip(("q", "k", "v"), O.attention_backward(f64(q), f64(k), f64(v), 0.125, f64(do), f64(mask))):
        assert_close(arrays["gradient_" + name], w, torch.float16, "d" + name, atol=1e-2 * max(1.0, float(np.abs(w).max())))


# ----------------------------------------------------------------------------- MBConv block
def _mbconv(seed=4, b=3, cin=16, hw=28, cout=24):
    from daceml_amd import graphs
    r = rng(seed)
    sdfg = graphs.mbconv_block(b, cin, hw, expand=6, cout=cout, se_reduce=4, stride=2, dtype=torch.float32)
    x = r.standard_normal((b, cin, hw, hw)).astype(np.float32)
    params = {}
    for name, desc in sdfg.arglist().items():
        if name in ("x", "y"):
            continue
        if name.endswith("_w"):
            fan_in = int(np.prod(desc.shape[1:]))
            params[name] = (r.standard_normal(desc.shape) * np.sqrt(2.0 / fan_in)).astype(np.float32)
        else:
            params[name] = (r.standard_normal(desc.shape) * 0.1).astype(np.float32)
    return sdfg, x, params


def _mbconv_reference(x, p, dy=None):
    """The block in torch, fp64 (its structure: expand 1x1 + swish, depthwise 3x3 stride 2 + swish, squeeze-excite,
    project 1x1), with autograd for the gradients."""
    import torch.nn.functional as F
    t = {k: torch.tensor(v.astype(np.float64), requires_grad=True) for k, v in p.items()}
    xt = torch.tensor(x.astype(np.float64), requires_grad=True)
    sw = lambda v: v * torch.sigmoid(v)  # noqa: E731
    h = sw(F.conv2d(xt, t["expand_w"], t["expand_b"]))
    h = sw(F.conv2d(h, t["dw_w"], t["dw_b"], stride=2, padding=1, groups=h.shape[1]))
    g = h.mean((2, 3), keepdim=True)
    g = torch.sigmoid(F.conv2d(sw(F.conv2d(g, t["se1_w"], t["se1_b"])), t["se2_w"], t["se2_b"]))
    y = F.conv2d(h * g, t["proj_w"], t["proj_b"])
    grads = None
    if dy is not None:
        y.backward(torch.tensor(dy.astype(np.float64)))
        grads = {"x": xt.grad.numpy(), **{k: v.grad.numpy() for k, v in t.items()}}
    return y.detach().numpy(), grads


@pytest.mark.parametrize("fused", [False, True])
def test_mbconv_block_forward(fused):
    import copy
    from daceml_amd.runtime import expand_onnx_nodes
    from daceml_amd.transformation import fusion
    sdfg, x, p = _mbconv(cin=16, hw=28)
    want, _ = _mbconv_reference(x, p)
    if fused:
        stats = fusion.auto_optimize(sdfg)
        assert stats["gated_conv"] == 1 and stats["expand_depthwise"] == 1
    expand_onnx_nodes(sdfg)
    arrays = {"x": x.copy(), **copy.deepcopy(p)}
    log = run_sdfg(sdfg, arrays)
    if fused:
        assert "dmlhip_conv2d_expand_depthwise_f32" in log and "dmlhip_conv2d_gated_f32" in log
    assert_close(arrays["y"], want, torch.float32, "mbconv forward fused=%s" % fused, rtol=1e-4, atol=1e-5)


def test_mbconv_block_training_step():
    import copy
    from daceml_amd.autodiff import add_backward_pass
    from daceml_amd.runtime import expand_onnx_nodes
    from daceml_amd.transformation import fusion
    sdfg, x, p = _mbconv(cin=16, hw=28)
    fusion.auto_optimize(sdfg, training=True)
    wrt = ["x"] + sorted(p)
    grads = add_backward_pass(sdfg, sdfg.states()[0], ["y"], wrt)
    fusion.optimize_backward(sdfg)
    expand_onnx_nodes(sdfg)
    dy = rng(6).standard_normal(tuple(sdfg.arrays["y"].shape)).astype(np.float32)
    arrays = {"x": x.copy(), "gradient_y": dy.copy(), **copy.deepcopy(p)}
    run_sdfg(sdfg, arrays)
    want_y, want = _mbconv_reference(x, p, dy)
    assert_close(arrays["y"], want_y, torch.float32, "mbconv training forward", rtol=1e-4, atol=1e-5)
    for n in wrt:
        scale = max(1.0, float(np.abs(want[n]).max()))
        assert_close(arrays[grads[n]], want[n], torch.float32, "mbconv d" + n, rtol=1e-4, atol=1e-5 * scale)


# ----------------------------------------------------------------------------- an exported module in training mode
def test_conv_batchnorm_relu_module_training_step():
    """torch.nn.Conv2d -> BatchNorm2d -> ReLU in training mode through the exporter, the importer, the fusion passes
    (the ReLU moves into the normalisation kernels) and the autodiff generator, interpreted on the CPU: output, input
    and parameter gradients against autograd in fp64, and the running statistics the forward call leaves behind."""
    import copy
    from daceml_amd.autodiff import add_backward_pass
    from daceml_amd.onnx.onnx_importer import clean_onnx_name
    from daceml_amd.runtime import expand_onnx_nodes
    from daceml_amd.torch import DaceModule
    from daceml_amd.transformation import fusion
    torch.manual_seed(11)
    net = torch.nn.Sequential(torch.nn.Conv2d(3, 8, 3, padding=1), torch.nn.BatchNorm2d(8), torch.nn.ReLU())
    with torch.no_grad():
        net[1].weight.uniform_(0.5, 1.5)
        net[1].bias.normal_(0, 0.2)
        net[1].running_mean.normal_(0, 0.3)
        net[1].running_var.uniform_(0.5, 2.0)
    ref = copy.deepcopy(net).double().train()
    x = torch.randn(4, 3, 10, 10)
    wrapped = DaceModule(copy.deepcopy(net).train(), training=True, backward=True)
    model = wrapped._import((x, ))
    sdfg, state = model.sdfg, model.state
    names = [n.schema.name for n in state.library_nodes()]
    assert names == ["Conv", "BatchNormalization"] and state.library_nodes()[1]._activation == "relu"
    fusion.lower_matmul(sdfg)
    params = dict(net.named_parameters())
    wrt = [clean_onnx_name(n) for n in model.inputs if n == model.inputs[0] or n in params]
    grads = add_backward_pass(sdfg, state, list(model.outputs), wrt)
    fusion.optimize_backward(sdfg)
    expand_onnx_nodes(sdfg)
    state_dict = {**params, **dict(net.named_buffers())}
    arrays = {clean_onnx_name(model.inputs[0]): x.numpy().copy()}
    for n in model.inputs[1:]:
        arrays[clean_onnx_name(n)] = state_dict[n].detach().numpy().copy()
    dy = torch.randn(4, 8, 10, 10)
    arrays["gradient_" + model.outputs[0]] = dy.numpy().copy()
    log = run_sdfg(sdfg, arrays)
    assert any(s_.startswith("dmlhip_batchnorm_training_act") for s_ in log)
    assert any(s_.startswith("dmlhip_batchnorm_backward_act") for s_ in log)
    xr = x.double().requires_grad_(True)
    want = ref(xr)
    want.backward(dy.double())
    assert_close(arrays[model.outputs[0]], want.detach().numpy(), torch.float32, "training forward", rtol=1e-4, atol=1e-5)
    assert_close(arrays[grads[clean_onnx_name(model.inputs[0])]], xr.grad.numpy(), torch.float32, "dx", rtol=1e-4, atol=1e-5)
    for n, pr in ref.named_parameters():
        scale = max(1.0, float(pr.grad.abs().max()))
        assert_close(arrays[grads[clean_onnx_name(n)]], pr.grad.numpy(), torch.float32, "gradient of " + n, rtol=1e-4,
                     atol=1e-5 * scale)
    # running statistics: torch blends the unbiased batch variance, the reference (and the kernels) the biased one
    # (img_op_implementations.py:373-390); the mean follows the same rule in both
    assert_close(arrays[clean_onnx_name("1.running_mean")], ref[1].running_mean.numpy(), torch.float32, "running mean",
                 rtol=1e-4, atol=1e-6)
    count = 4 * 10 * 10
    biased = (ref[1].running_var.numpy() - 0.9 * net[1].running_var.numpy()) / 0.1 * (count - 1) / count
    assert_close(arrays[clean_onnx_name("1.running_var")], 0.9 * net[1].running_var.numpy() + 0.1 * biased, torch.float32,
                 "running variance", rtol=1e-4, atol=1e-6)
