"""Fused attention with an additive mask (the Add that a BERT encoder's export places between the scaled scores and the
Softmax; pure_implementations.py:34-36, 309-319).

The host-side tests run everywhere: the fusion pass recognises the chain, the expansions emit the masked entry points
with the right strides, the gradient node receives the mask. The GPU tests compare the kernels with
``oracle.ops.attention(..., mask)`` (the kernels without a mask are separate instantiations)."""
import numpy as np
import pytest
import torch

from oracle import ops as O
from tests.util import assert_close, dev, host, rng



# ----------------------------------------------------------------------------- host side
def _chain(mask_shape, mask_dtype=torch.float16, b=2, h=3, sq=40, sk=48, mask_first=False, scale_op="Mul"):
    """scores = Einsum(q, k) * scale; scores + mask; Softmax; Einsum(p, v) - as the exporter emits it."""
    from daceml_amd import graphs
    g = graphs.GraphBuilder("attn", torch.float16)
    q, k, v = g.input("q", (b, h, sq, 64)), g.input("k", (b, h, sk, 64)), g.input("v", (b, h, sk, 64))
    m = g.input("mask", mask_shape, dtype=mask_dtype) if mask_dtype != torch.float16 else g.input("mask", mask_shape)
    s = g.node("Einsum", {"Inputs__0": q, "Inputs__1": k}, {"Output": (b, h, sq, sk)}, label="scores",
               equation="bhqd,bhkd->bhqk")["Output"]
    c = g.constant("scale", np.array(0.125 if scale_op == "Mul" else 8.0, dtype=np.float16))
    s = g.node(scale_op, {"A": s, "B": c}, {"C": (b, h, sq, sk)}, label="scale")["C"]
    s = g.node("Add", {"A": m, "B": s} if mask_first else {"A": s, "B": m}, {"C": (b, h, sq, sk)}, label="mask")["C"]
    p = g.node("Softmax", {"input": s}, {"output": (b, h, sq, sk)}, label="softmax", axis=-1)["output"]
    o = g.node("Einsum", {"Inputs__0": p, "Inputs__1": v}, {"Output": (b, h, sq, 64)}, label="context",
               equation="bhqk,bhkd->bhqd")["Output"]
    g.output(o, "o")
    return g


def _fused(g):
    from daceml_amd.transformation import fusion
    fusion.auto_optimize(g.sdfg)
    return [n for n in g.state.library_nodes() if n.schema.name == "FusedAttention"]


@pytest.mark.parametrize("mask_shape,strides", [((2, 1, 1, 48), (48, 0)), ((1, 1, 1, 48), (0, 0)), ((2, 3, 1, 48), (144, 48)),
                                                ((1, 3, 1, 48), (0, 48)), ((48, ), (0, 0)), ((1, 48), (0, 0))])
@pytest.mark.parametrize("mask_first", [False, True])
def test_masked_chain_becomes_one_node_with_the_mask_as_input(mask_shape, strides, mask_first):
    g = _chain(mask_shape, mask_first=mask_first)
    nodes = _fused(g)
    assert len(nodes) == 1 and [n.schema.name for n in g.state.library_nodes()] == ["FusedAttention"]
    node = nodes[0]
    assert {e.dst_conn: e.data.data for e in g.state.in_edges(node)} == {"Q": "q", "K": "k", "V": "v", "Mask": "mask"}
    assert abs(node.scale - 0.125) < 1e-6
    t = node.expand(g.sdfg, g.state)
    assert [c.symbol for c in t.calls] == ["dmlhip_attention_masked_f16"]
    from daceml_amd import hip_tasklet as T
    arrays = [a for a in t.calls[0].args if isinstance(a, T.I64Array)]
    assert len(arrays) == 1 and tuple(arrays[0].values) == strides


@pytest.mark.parametrize("mask_shape,dtype", [((2, 1, 40, 48), torch.float16),     # varies with the query
                                              ((2, 3, 40, 48), torch.float16),
                                              ((2, 1, 1, 48), torch.float32)])     # not the tensors' type
def test_masks_the_kernels_cannot_take_leave_the_chain_alone(mask_shape, dtype):
    g = _chain(mask_shape, mask_dtype=dtype)
    assert _fused(g) == []
    names = [n.schema.name for n in g.state.library_nodes()]
    # (a mask of the scores' own shape is folded into the first contraction as its residual operand instead)
    assert "Softmax" in names and ("Add" in names or tuple(mask_shape) == (2, 3, 40, 48))


def test_mask_rows_that_are_not_eight_byte_aligned_are_refused():
    # 50 keys: rows of a [2, 1, 1, 50] mask start at odd multiples of 4 bytes
    g = _chain((2, 1, 1, 50), sk=50)
    assert _fused(g) == []
    g = _chain((1, 1, 1, 50), sk=50)      # a single row has no stride to align
    assert len(_fused(g)) == 1


def test_gradient_node_gets_the_mask_and_the_mask_gets_no_gradient():
    from daceml_amd.autodiff import add_backward_pass
    from daceml_amd.autodiff.base_abc import AutoDiffException
    g = _chain((2, 1, 1, 48))
    assert len(_fused(g)) == 1
    grads = add_backward_pass(g.sdfg, g.state, ["o"], ["q", "k", "v"])
    assert set(grads) == {"q", "k", "v"}
    bst = g.sdfg.states()[1]
    gn = [n for n in bst.library_nodes() if n.schema.name == "FusedAttentionGrad"]
    assert len(gn) == 1
    assert {e.dst_conn: e.data.data for e in bst.in_edges(gn[0])}["Mask"] == "mask"
    t = gn[0].expand(g.sdfg, bst)
    assert [c.symbol for c in t.calls] == ["dmlhip_attention_masked_backward_f16"]
    g2 = _chain((2, 1, 1, 48))
    _fused(g2)
    with pytest.raises(AutoDiffException):
        add_backward_pass(g2.sdfg, g2.state, ["o"], ["q", "mask"])


def test_argument_errors_of_the_masked_entry_points(lib):
    """Checked before anything is launched: NULL mask, misaligned mask, strides that are not multiples of four."""
    import ctypes
    from daceml_amd import _lib as L
    d = L.AttentionDesc()
    d.batch[0], d.batch[1], d.seq_q, d.seq_k, d.head_dim, d.scale = 1, 1, 64, 64, 64, 0.125
    for name in ("q_stride", "k_stride", "v_stride", "o_stride"):
        getattr(d, name)[0], getattr(d, name)[1], getattr(d, name)[2] = 4096, 4096, 64
    ms = (ctypes.c_int64 * 2)(0, 0)
    buf = 1 << 20   # a fake, aligned, non-NULL address: argument checks come first and nothing is dereferenced
    assert lib.dmlhip_attention_masked_f16(ctypes.byref(d), buf, buf, buf, None, ms, buf, None, None) == L.ERR_NULL
    assert lib.dmlhip_attention_masked_f16(ctypes.byref(d), buf, buf, buf, buf, None, buf, None, None) == L.ERR_NULL
    assert lib.dmlhip_attention_masked_f16(ctypes.byref(d), buf, buf, buf, buf + 2, ms, buf, None, None) == L.ERR_ALIGN
    bad = (ctypes.c_int64 * 2)(66, 0)
    assert lib.dmlhip_attention_masked_f16(ctypes.byref(d), buf, buf, buf, buf, bad, buf, None, None) == L.ERR_ALIGN
    neg = (ctypes.c_int64 * 2)(0, -4)
    assert lib.dmlhip_attention_masked_f16(ctypes.byref(d), buf, buf, buf, buf, neg, buf, None, None) == L.ERR_ALIGN
    assert b"mask" in lib.dmlhip_last_error_string()


# ----------------------------------------------------------------------------- kernels (GPU)
def _mask(seed, b0, b1, sk, kind):
    """(device tensor, float64 array). `kind`: which batch dims the mask has, and what it holds."""
    r = rng(seed)
    per_head = "h" in kind
    shape = (b0, b1 if per_head else 1, 1, sk)
    if "pad" in kind:       # BERT's padding mask: 0 for real tokens, -10000 behind a per-batch length
        m = np.zeros(shape, np.float16)
        for b in range(b0):
            m[b, :, :, max(1, sk - 1 - (b * 7 + 3) % sk):] = -10000.0
    elif "inf" in kind:
        m = np.zeros(shape, np.float16)
        m[..., sk // 2:] = -np.inf
    else:                   # a bias of ordinary size
        m = (r.standard_normal(shape) * 2).astype(np.float16)
    # rows padded to a multiple of four elements, as the entry point wants them
    pitch = (sk + 3) // 4 * 4
    base = torch.zeros(shape[:3] + (pitch, ), dtype=torch.float16, device="cuda")
    base[..., :sk] = dev(m)
    return base[..., :sk], m.astype(np.float64)


MASK_CASES = [(2, 3, 128, 128, "pad"), (2, 2, 100, 77, "pad"), (1, 2, 512, 512, "bias"), (2, 3, 64, 321, "h-bias"),
              (1, 1, 1, 1, "bias"), (2, 1, 257, 64, "h-pad"), (2, 2, 70, 200, "inf"), (1, 3, 33, 130, "h-bias")]


@pytest.mark.gpu
@pytest.mark.parametrize("layout", ["bhsd", "bshd"])
@pytest.mark.parametrize("b0,b1,sq,sk,kind", MASK_CASES)
def test_masked_attention_forward_and_backward(b0, b1, sq, sk, kind, layout):
    from daceml_amd import kernels as K
    from tests.test_gpu_kernels import _attn_tensor
    q, q64 = _attn_tensor(170, b0, b1, sq, layout)
    k, k64 = _attn_tensor(171, b0, b1, sk, layout)
    v, v64 = _attn_tensor(172, b0, b1, sk, layout)
    do, do64 = _attn_tensor(173, b0, b1, sq, layout)
    mask, m64 = _mask(174, b0, b1, sk, kind)
    scale = 0.125
    out, lse = K.attention(q, k, v, scale, mask=mask)
    want, want_lse = O.attention(q64, k64, v64, scale, m64)
    what = str((b0, b1, sq, sk, kind, layout))
    assert_close(host(out), want, torch.float16, "masked attention " + what)
    assert_close(host(lse), want_lse, torch.float32, "masked attention lse " + what, rtol=1e-3, atol=1e-3)
    dq, dk, dv = K.attention_backward(q, k, v, out, lse, do, scale, mask=mask)
    for name, got, w in zip(("dq", "dk", "dv"), (dq, dk, dv), O.attention_backward(q64, k64, v64, scale, do64, m64)):
        s = max(1.0, float(np.abs(w).max()))
        assert_close(host(got), w, torch.float16, "masked attention backward %s %s" % (name, what), atol=1e-2 * s)
    if kind == "inf":   # keys at -inf take no part: no gradient reaches them
        assert float(dk[:, :, sk // 2:].abs().max()) == 0.0 and float(dv[:, :, sk // 2:].abs().max()) == 0.0
    # a mask of zeros is the kernel without a mask up to rounding (the masked kernel rounds scale * s + mask before it
    # subtracts the row maximum, the plain one fuses the two): a few fp16 units in the last place
    zero = torch.zeros(tuple(mask.shape[:3]) + ((sk + 3) // 4 * 4, ), dtype=torch.float16, device="cuda")[..., :sk]
    out0, lse0 = K.attention(q, k, v, scale, mask=zero)
    out1, lse1 = K.attention(q, k, v, scale)
    assert_close(host(out0), host(out1), torch.float16, "zero mask " + what, rtol=4e-3, atol=5e-4)
    assert_close(host(lse0), host(lse1), torch.float32, "zero mask lse " + what, rtol=1e-5, atol=1e-5)


class _MaskedBert(torch.nn.Module):
    def __init__(self, layer):
        super().__init__()
        self.layer = layer

    def forward(self, x, mask):
        out = self.layer(x, attention_mask=mask)
        return out[0] if isinstance(out, (tuple, list)) else out


def _bert_layer(hidden=128, heads=2, ffn=256):
    transformers = pytest.importorskip("transformers")
    from transformers.models.bert.modeling_bert import BertConfig, BertLayer
    cfg = BertConfig(hidden_size=hidden, num_attention_heads=heads, intermediate_size=ffn, hidden_dropout_prob=0.0,
                     attention_probs_dropout_prob=0.0)
    try:
        cfg._attn_implementation = "eager"
    except Exception:
        pass
    torch.manual_seed(0)
    del transformers
    return _MaskedBert(BertLayer(cfg).eval())


def test_exported_bertlayer_with_attention_mask_is_fused_on_import():
    """HuggingFace's BertLayer called with the extended attention mask [batch, 1, 1, keys] (the module the reference's
    own integration test wraps, tests/torch/test_bert_encoder.py:13-19, there without a mask): exported in fp16,
    imported and optimised without a GPU, the attention block is one node that reads the mask input."""
    from daceml_amd.torch import DaceModule
    net = _bert_layer().half()
    x = torch.randn(2, 48, 128).half()
    mask = torch.zeros(2, 1, 1, 48).half()
    mask[1, :, :, 30:] = -10000.0
    model = DaceModule(net)._import((x, mask))
    st = model.sdfg.states()[0]
    names = [n.schema.name for n in st.library_nodes()]
    assert names.count("FusedAttention") == 1 and "Softmax" not in names and "Add" not in names
    node = [n for n in st.library_nodes() if n.schema.name == "FusedAttention"][0]
    ins = {e.dst_conn: e.data.data for e in st.in_edges(node)}
    assert ins["Mask"] == "attention_mask" and abs(node.scale - 0.125) < 1e-6
    t = node.expand(model.sdfg, st)
    assert [c.symbol for c in t.calls] == ["dmlhip_attention_masked_f16"]


@pytest.mark.gpu
def test_huggingface_bertlayer_with_attention_mask_stays_on_the_fused_path():
    from daceml_amd.torch import DaceModule
    net = _bert_layer().half().cuda()
    x = torch.randn(2, 48, 128, device="cuda").half()
    mask = torch.zeros(2, 1, 1, 48, device="cuda").half()
    mask[1, :, :, 30:] = -10000.0
    # as with the reference's wrapper, every floating-point input gets a gradient unless it is listed here
    # (daceml/torch/module.py:333-346); the fused attention node produces none for its mask
    wrapped = DaceModule(net, backward=True, inputs_to_skip=["attention_mask"])
    xg = x.clone().requires_grad_(True)
    got = wrapped(xg, mask)
    symbols = [l.symbol for l in wrapped.compiled.launches]
    assert "dmlhip_attention_masked_f16" in symbols and not any("softmax" in s for s in symbols)
    ref = _bert_layer().double().cuda()
    ref.load_state_dict({k_: v_.double() for k_, v_ in net.state_dict().items()})
    xr = x.double().requires_grad_(True)
    want = ref(xr, mask.double())
    assert_close(host(got), want.detach().cpu().numpy(), torch.float16, "BertLayer with mask")
    dy = torch.randn_like(got)
    got.backward(dy)
    want.backward(dy.double())
    assert_close(host(xg.grad), xr.grad.cpu().numpy(), torch.float16, "BertLayer with mask: input gradient", atol=2e-2)
