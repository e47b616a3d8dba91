"""GPU parity of whole graphs run through the library-node registry, the fusion pass, the autodiff
registry and the runtime: BERT encoder layer forward / backward and the MBConv block, against the NumPy
oracle on the same seeded inputs."""
import numpy as np
import pytest
import torch

from oracle import bert_layer as OB
from oracle import ops as O
from tests.util import assert_close, dev, host, rng

pytestmark = pytest.mark.gpu


def _bert_inputs(b, s, h, ffn, dtype, seed=1234, bias_std=0.02):
    npdt = np.float16 if dtype == torch.float16 else np.float32
    p = OB.init_params(h, ffn, seed, np.float32, bias_std=bias_std)
    r = rng(seed + 1)
    p["ln1_g"] = r.uniform(0.5, 1.5, h).astype(np.float32)
    p["ln2_g"] = r.uniform(0.5, 1.5, h).astype(np.float32)
    p["ln1_b"] = (r.standard_normal(h) * 0.1).astype(np.float32)
    p["ln2_b"] = (r.standard_normal(h) * 0.1).astype(np.float32)
    x = r.standard_normal((b, s, h)).astype(np.float32)
    p = {k: v.astype(npdt) for k, v in p.items()}
    return x.astype(npdt), p


def _compile(sdfg, reuse_transients=False):
    from daceml_amd.runtime import CompiledSDFG
    return CompiledSDFG(sdfg, reuse_transients=reuse_transients)


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
@pytest.mark.parametrize("fused", ["attention", True, False])
def test_bert_layer_forward(dtype, fused):
    from daceml_amd import graphs
    from daceml_amd.transformation import fusion
    b, s, h, heads, ffn = 2, 128, 256, 4, 1024
    x, p = _bert_inputs(b, s, h, ffn, dtype)
    sdfg = graphs.bert_encoder_layer(b, s, h, heads, ffn, dtype, eps=1e-5)
    if fused:
        # "attention": the default pipeline (fused attention, Gelu as its own kernel); True: Gelu in the GEMM epilogue
        stats = fusion.auto_optimize(sdfg, attention=fused == "attention", gelu_epilogue=fused is True)
        assert stats["layernorm"] == 2 and stats["gelu"] == 1 and stats["epilogues"] == 7
        names = [n.schema.name for n in sdfg.states()[0].library_nodes()]
        if fused == "attention" and dtype == torch.float16:  # the fused kernel is fp16 only
            assert stats["attention"] == 1
            assert sorted(set(names)) == ["FusedAttention", "FusedEinsum", "Gelu", "GroupedEinsum", "LayerNormalization"]
        else:
            assert stats["attention"] == 0
            extra = ["Gelu"] if fused == "attention" else []
            # the three projections run as one grouped launch where the grouped kernel exists (fp16)
            extra += ["GroupedEinsum"] if dtype == torch.float16 else []
            assert sorted(set(names)) == sorted(["Einsum", "FusedEinsum", "LayerNormalization", "Softmax"] + extra)
    prog = _compile(sdfg)
    y = torch.empty((b, s, h), dtype=dtype, device="cuda")
    prog(x=dev(x), y=y, **{k: dev(v) for k, v in p.items()})
    want = OB.forward(x.astype(np.float64), {k: v.astype(np.float64) for k, v in p.items()}, heads, eps=1e-5)
    if dtype == torch.float16:
        assert_close(host(y), want, dtype, "bert layer forward fused=%s" % fused)
    else:
        # a chain of ~12 fp32 nodes with K up to 1024: rounding accumulates beyond one node's 1e-5 / 1e-6
        assert_close(host(y), want, dtype, "bert layer forward fused=%s" % fused, rtol=1e-4, atol=2e-5)


@pytest.mark.parametrize("reuse", [False, True], ids=["own_buffers", "arena"])
@pytest.mark.parametrize("dtype,attention", [(torch.float16, True), (torch.float16, False), (torch.float32, False)])
def test_bert_layer_backward(dtype, attention, reuse):
    """``reuse``: the transients share one arena by lifetime (and the launch order is the one chosen for a small memory
    peak), as in the benchmarked program."""
    from daceml_amd import graphs
    from daceml_amd.autodiff import add_backward_pass
    from daceml_amd.transformation import fusion
    b, s, h, heads, ffn = 2, 128, 256, 4, 1024
    x, p = _bert_inputs(b, s, h, ffn, dtype)
    dy = rng(77).standard_normal((b, s, h)).astype(x.dtype)
    sdfg = graphs.bert_encoder_layer(b, s, h, heads, ffn, dtype, eps=1e-5)
    fusion.auto_optimize(sdfg, training=True, attention=attention, gelu_epilogue=not attention)
    grads = add_backward_pass(sdfg, sdfg.states()[0], ["y"], ["x"] + OB.PARAM_NAMES,
                              grad_dtypes={n: torch.float32 for n in OB.PARAM_NAMES})
    if attention:
        assert fusion.optimize_backward(sdfg)["bias_gradients"] == 6   # produced by the weight-gradient contractions
    # the backward state contains only nodes with hand-written kernels
    bnames = {n.schema.name for n in sdfg.states()[1].library_nodes()}
    if attention:
        assert bnames == {"FusedEinsum", "GroupedEinsum", "EinsumSum", "FusedAttentionGrad", "LayerNormalizationGrad",
                          "GeluGrad"}
    else:
        assert bnames == {"FusedEinsum", "SoftmaxGrad", "LayerNormalizationGrad", "GeluGrad", "ReduceSum", "Sum"}
    n_grouped = sum(n.schema.name in ("GroupedEinsum", "EinsumSum") or "InputSum" in n.out_connectors
                    for st in sdfg.states() for n in st.library_nodes())
    prog = _compile(sdfg, reuse)   # expands the library nodes in place
    if reuse:
        own = sum(t.numel() * t.element_size() for n, t in prog.buffers.items() if sdfg.arrays[n].transient)
        assert 0 < prog.arena_bytes < 0.7 * own
    args = {"x": dev(x), "y": torch.empty((b, s, h), dtype=dtype, device="cuda"), "gradient_y": dev(dy)}
    args.update({k: dev(v) for k, v in p.items()})
    out = {"gradient_x": torch.empty((b, s, h), dtype=dtype, device="cuda")}
    for n in OB.PARAM_NAMES:
        out["gradient_" + n] = torch.empty(p[n].shape, dtype=torch.float32, device="cuda")
    from daceml_amd import _lib
    single = _lib.load().dmlhip_debug_grouped_single_launches
    before = single()
    prog(**args, **out)
    if attention:
        # q/k/v projections, the sum of their input gradients and the o/q/k/v weight gradients: one launch each, also
        # for the two backward nodes, which carry no bias table
        # (plus the two FFN weight gradients that produce their bias gradient alongside)
        assert n_grouped == 5 and single() - before == 5
    x64 = x.astype(np.float64)
    p64 = {k: v.astype(np.float64) for k, v in p.items()}
    _, saved = OB.forward(x64, p64, heads, eps=1e-5, keep=True)
    want = OB.backward(x64, p64, heads, dy.astype(np.float64), saved, eps=1e-5, term_scales=True)
    assert grads["x"] == "gradient_x"
    if dtype == torch.float16:
        assert_close(host(out["gradient_x"]), want["x"], dtype, "dx")
        for n in OB.PARAM_NAMES:
            # fp32 master gradients: sums over the rows of products of tensors stored in fp16. On top of the stated
            # tolerance an element is allowed 16 x 2^-11 x the root of the sum of squares of its exact terms (the key
            # bias has an exactly zero gradient - softmax is shift invariant - and what is left there is the rounding
            # of the values that cancel)
            assert_close(host(out["gradient_" + n]), want[n], dtype, "d" + n, rtol=2e-2,
                         atol=1e-2 + 16.0 * 2.0 ** -11 * want["terms:" + n])
    else:
        assert_close(host(out["gradient_x"]), want["x"], dtype, "dx", rtol=1e-4, atol=2e-5)
        for n in OB.PARAM_NAMES:
            scale = float(np.abs(want[n]).max())
            assert_close(host(out["gradient_" + n]), want[n], dtype, "d" + n, rtol=1e-4, atol=1e-5 * max(scale, 1.0))


def test_mbconv_block_forward():
    from daceml_amd import graphs
    from daceml_amd.transformation import fusion
    b, cin, hw, cout = 3, 16, 28, 24
    r = rng(4)
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
    stats = fusion.auto_optimize(sdfg)
    assert stats["swish"] == 3 and stats["conv_activation"] == 4 and stats["gated_conv"] == 1
    assert stats["expand_depthwise"] == 1
    names = [n.schema.name for n in sdfg.states()[0].library_nodes()]
    assert names.count("GatedConv") == 1 and "Mul" not in names   # the squeeze-excite Mul went into the projection
    assert names.count("ExpandDepthwiseConv") == 1                # the expanded tensor stays on chip
    prog = _compile(sdfg)
    oh = (hw + 2 - 3) // 2 + 1
    y = torch.empty((b, cout, oh, oh), dtype=torch.float32, device="cuda")
    prog(x=dev(x), y=y, **{k: dev(v) for k, v in params.items()})
    # oracle: the unfused node sequence
    f = {k: v.astype(np.float64) for k, v in params.items()}
    t = O.swish(O.conv2d(x.astype(np.float64), f["expand_w"], f["expand_b"]))
    t = O.swish(O.conv2d(t, f["dw_w"], f["dw_b"], strides=(2, 2), pads=(1, 1, 1, 1), group=cin * 6))
    se = O.global_average_pool(t)
    se = O.swish(O.conv2d(se, f["se1_w"], f["se1_b"]))
    se = O.sigmoid(O.conv2d(se, f["se2_w"], f["se2_b"]))
    want = O.conv2d(O.mul(t, se), f["proj_w"], f["proj_b"])
    # the reference's own tolerance for this block is 1e-3 (tests/torch/test_efficientnet_block.py:50-54);
    # five chained fp32 nodes hold 1e-5 relative with a slightly wider absolute floor
    assert_close(host(y), want, torch.float32, "mbconv forward", rtol=1e-5, atol=5e-6)


def test_selection_levels_and_refusal():
    """node.implementation > class default > package default; an inapplicable node raises, it does not
    fall back silently."""
    import daceml_amd.onnx as donnx
    from daceml_amd.runtime import expand_onnx_nodes
    from daceml_amd.sdfg import SDFG
    sdfg = SDFG("t")
    st = sdfg.add_state()
    sdfg.add_array("a", (4, 8), torch.float16)
    sdfg.add_array("b", (4, 8), torch.float16)
    node = donnx.ONNXSoftmax("sm", axis=-1)
    st.add_edge(st.add_read("a"), None, node, "input", sdfg.make_array_memlet("a"))
    st.add_edge(node, "output", st.add_write("b"), None, sdfg.make_array_memlet("b"))
    node.implementation = "does-not-exist"
    with pytest.raises(donnx.NotApplicable):
        expand_onnx_nodes(sdfg)
    node.implementation = None
    assert expand_onnx_nodes(sdfg) == 1


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
def test_elementwise_backward_with_broadcast(dtype):
    """Mul / Sub / Div reversed as elementwise nodes plus a reduction for the broadcast operand (what the reference
    gets from symbolic tasklet reversal and ReverseReduce), against autograd."""
    from daceml_amd import graphs
    from daceml_amd.autodiff import add_backward_pass
    g = graphs.GraphBuilder("elementwise_backward", dtype)
    a, b, c = g.input("a", (6, 5, 32)), g.input("b", (32, )), g.input("c", (6, 5, 32))
    m = g.node("Mul", {"A": a, "B": b}, {"C": (6, 5, 32)}, label="m")["C"]
    s_ = g.node("Sub", {"A": m, "B": c}, {"C": (6, 5, 32)}, label="s")["C"]
    d = g.node("Div", {"A": s_, "B": b}, {"C": (6, 5, 32)}, label="d")["C"]
    t = g.node("Sub", {"A": b, "B": d}, {"C": (6, 5, 32)}, label="t")["C"]     # broadcast operand first
    g.output(t, "y")
    grads = add_backward_pass(g.sdfg, g.state, ["y"], ["a", "b", "c"])
    assert grads == {"a": "gradient_a", "b": "gradient_b", "c": "gradient_c"}
    prog = _compile(g.sdfg)
    npdt = np.float16 if dtype == torch.float16 else np.float32
    av = rng(1).standard_normal((6, 5, 32)).astype(npdt)
    bv = (rng(2).uniform(0.5, 1.5, 32)).astype(npdt)
    cv = rng(3).standard_normal((6, 5, 32)).astype(npdt)
    dyv = rng(4).standard_normal((6, 5, 32)).astype(npdt)
    out = {n: torch.empty(s, dtype=dtype, device="cuda") for n, s in
           (("y", (6, 5, 32)), ("gradient_a", (6, 5, 32)), ("gradient_b", (32, )), ("gradient_c", (6, 5, 32)))}
    prog(a=dev(av), b=dev(bv), c=dev(cv), gradient_y=dev(dyv), **out)
    ta, tb, tc = (torch.tensor(v.astype(np.float64), requires_grad=True) for v in (av, bv, cv))
    ty = tb - (ta * tb - tc) / tb
    ty.backward(torch.tensor(dyv.astype(np.float64)))
    assert_close(host(out["y"]), ty.detach().numpy(), dtype, "forward")
    for name, want in (("a", ta.grad), ("b", tb.grad), ("c", tc.grad)):
        kw = dict(rtol=1e-4, atol=1e-4) if dtype == torch.float32 else dict(atol=0.1 if name == "b" else 1e-2)
        assert_close(host(out["gradient_" + name]), want.numpy(), dtype, "gradient of " + name, **kw)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
def test_unfused_layernorm_and_gelu_chains_backward(dtype):
    """The exporter's decomposed LayerNormalization (ReduceMean, Sub, Pow, ReduceMean, Add, Sqrt, Div, Mul, Add) and GELU
    (Div, Erf, Add, Mul, Mul) differentiated node by node, without the fusion pass (the reference reverses these maps
    symbolically, backward_pass_generator.py:1284-1421), against autograd on the same expression."""
    from daceml_amd import graphs
    from daceml_amd.autodiff import add_backward_pass
    g = graphs.GraphBuilder("chains_backward", dtype)
    x = g.input("x", (3, 7, 64))
    g.input("gamma", (64, ))
    g.input("beta", (64, ))
    ln = g.layer_norm(x, "gamma", "beta", 1e-5, "ln")
    g.output(g.gelu(ln, "act"), "y")
    grads = add_backward_pass(g.sdfg, g.state, ["y"], ["x", "gamma", "beta"])
    assert grads == {"x": "gradient_x", "gamma": "gradient_gamma", "beta": "gradient_beta"}
    kinds = [n.schema.name for n in g.sdfg.states()[1].library_nodes()]
    assert "ErfGrad" in kinds and "SqrtGrad" in kinds and kinds.count("ScaledExpand") == 2
    assert "LayerNormalizationGrad" not in kinds and "GeluGrad" not in kinds
    prog = _compile(g.sdfg)
    npdt = np.float16 if dtype == torch.float16 else np.float32
    xv = rng(21).standard_normal((3, 7, 64)).astype(npdt)
    gv = rng(22).uniform(0.5, 1.5, 64).astype(npdt)
    bv = (rng(23).standard_normal(64) * 0.1).astype(npdt)
    dyv = rng(24).standard_normal((3, 7, 64)).astype(npdt)
    out = {"y": torch.empty((3, 7, 64), dtype=dtype, device="cuda"),
           "gradient_x": torch.empty((3, 7, 64), dtype=dtype, device="cuda"),
           "gradient_gamma": torch.empty((64, ), dtype=dtype, device="cuda"),
           "gradient_beta": torch.empty((64, ), dtype=dtype, device="cuda")}
    prog(x=dev(xv), gamma=dev(gv), beta=dev(bv), gradient_y=dev(dyv), **out)
    tx, tg, tb = (torch.tensor(v.astype(np.float64), requires_grad=True) for v in (xv, gv, bv))
    ty = torch.nn.functional.gelu(torch.nn.functional.layer_norm(tx, (64, ), tg, tb, 1e-5))
    ty.backward(torch.tensor(dyv.astype(np.float64)))
    # fourteen chained elementwise / reduction nodes: every fp16 intermediate is rounded to fp16
    kw = dict(rtol=1e-4, atol=2e-5) if dtype == torch.float32 else dict(rtol=3e-2, atol=3e-2)
    assert_close(host(out["y"]), ty.detach().numpy(), dtype, "forward", **kw)
    assert_close(host(out["gradient_x"]), tx.grad.numpy(), dtype, "gradient of x", **kw)
    kw = dict(rtol=1e-4, atol=1e-4) if dtype == torch.float32 else dict(rtol=3e-2, atol=0.15)
    assert_close(host(out["gradient_gamma"]), tg.grad.numpy(), dtype, "gradient of gamma", **kw)
    assert_close(host(out["gradient_beta"]), tb.grad.numpy(), dtype, "gradient of beta", **kw)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
def test_squeeze_excite_gradient_meeting_point(dtype):
    """y = x * mean_hw(x): the gradient of x arrives through the multiplication and through the average pool. After
    optimize_backward the backward state is two kernels — the gate's gradient as a row-wise dot product and the sum of
    both paths as one RowAffine — checked against autograd."""
    from daceml_amd import graphs
    from daceml_amd.autodiff import add_backward_pass
    from daceml_amd.transformation import fusion
    g = graphs.GraphBuilder("se_meeting_point", dtype)
    x = g.input("x", (3, 5, 6, 8))
    gate = g.node("GlobalAveragePool", {"X": x}, {"Y": (3, 5, 1, 1)}, label="pool")["Y"]
    g.output(g.node("Mul", {"A": x, "B": gate}, {"C": (3, 5, 6, 8)}, label="scale")["C"], "y")
    assert add_backward_pass(g.sdfg, g.state, ["y"], ["x"]) == {"x": "gradient_x"}
    stats = fusion.optimize_backward(g.sdfg)
    assert stats["mul_reductions"] == 1 and stats["row_affine"] == 1
    assert sorted(n.schema.name for n in g.sdfg.states()[1].library_nodes()) == ["MulReduceSum", "RowAffine"]
    prog = _compile(g.sdfg)
    npdt = np.float16 if dtype == torch.float16 else np.float32
    xv = rng(31).standard_normal((3, 5, 6, 8)).astype(npdt)
    dyv = rng(32).standard_normal((3, 5, 6, 8)).astype(npdt)
    out = {"y": torch.empty((3, 5, 6, 8), dtype=dtype, device="cuda"),
           "gradient_x": torch.empty((3, 5, 6, 8), dtype=dtype, device="cuda")}
    prog(x=dev(xv), gradient_y=dev(dyv), **out)
    tx = torch.tensor(xv.astype(np.float64), requires_grad=True)
    ty = tx * tx.mean((2, 3), keepdim=True)
    ty.backward(torch.tensor(dyv.astype(np.float64)))
    kw = dict(rtol=1e-5, atol=2e-6) if dtype == torch.float32 else dict(rtol=2e-2, atol=2e-2)
    assert_close(host(out["y"]), ty.detach().numpy(), dtype, "forward", **kw)
    assert_close(host(out["gradient_x"]), tx.grad.numpy(), dtype, "gradient of x", **kw)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
def test_reduce_and_transpose_backward(dtype):
    """ReduceMean (keepdims 1), ReduceSum (keepdims 0) and Transpose reversed with ScaledExpand / Transpose nodes,
    against autograd: y = transpose(x - mean(x, -1, keepdim)) * sum(x, (0, 1))."""
    from daceml_amd import graphs
    from daceml_amd.autodiff import add_backward_pass
    g = graphs.GraphBuilder("reduce_backward", dtype)
    x = g.input("x", (4, 6, 16))
    mean = g.node("ReduceMean", {"data": x}, {"reduced": (4, 6, 1)}, label="mean", axes=[-1], keepdims=1)["reduced"]
    cen = g.node("Sub", {"A": x, "B": mean}, {"C": (4, 6, 16)}, label="cen")["C"]
    tr = g.node("Transpose", {"data": cen}, {"transposed": (6, 4, 16)}, label="tr", perm=[1, 0, 2])["transposed"]
    tot = g.node("ReduceSum", {"data": x}, {"reduced": (16, )}, label="tot", axes=[0, 1], keepdims=0)["reduced"]
    y = g.node("Mul", {"A": tr, "B": tot}, {"C": (6, 4, 16)}, label="scale")["C"]
    g.output(y, "y")
    assert add_backward_pass(g.sdfg, g.state, ["y"], ["x"]) == {"x": "gradient_x"}
    kinds = sorted(n.schema.name for n in g.sdfg.states()[1].library_nodes())
    assert kinds.count("ScaledExpand") == 2 and kinds.count("Transpose") == 1
    prog = _compile(g.sdfg)
    npdt = np.float16 if dtype == torch.float16 else np.float32
    xv = rng(11).standard_normal((4, 6, 16)).astype(npdt)
    dyv = rng(12).standard_normal((6, 4, 16)).astype(npdt)
    out = {"y": torch.empty((6, 4, 16), dtype=dtype, device="cuda"),
           "gradient_x": torch.empty((4, 6, 16), dtype=dtype, device="cuda")}
    prog(x=dev(xv), gradient_y=dev(dyv), **out)
    tx = torch.tensor(xv.astype(np.float64), requires_grad=True)
    ty = (tx - tx.mean(-1, keepdim=True)).permute(1, 0, 2) * tx.sum((0, 1))
    ty.backward(torch.tensor(dyv.astype(np.float64)))
    kw = dict(rtol=1e-4, atol=1e-4) if dtype == torch.float32 else dict(rtol=3e-2, atol=0.15)
    assert_close(host(out["y"]), ty.detach().numpy(), dtype, "forward", **kw)
    assert_close(host(out["gradient_x"]), tx.grad.numpy(), dtype, "gradient of x", **kw)

