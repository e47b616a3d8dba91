"""SDFGs of ONNX library nodes for the configurations the path is measured on, built node by node
the way DaCeML's importer builds them from a PyTorch opset-12 export
(daceml/onnx/onnx_importer.py:197-302; export settings daceml/torch/module.py:269-286: opset 12,
``do_constant_folding=False``, parameters kept as graph inputs).

Nothing is pre-fused here: ``nn.Linear`` is Transpose + MatMul + Add, ``nn.LayerNorm`` is the nine-node
ReduceMean ... Add chain, GELU is Div, Erf, Add, Mul, Mul, swish is Sigmoid + Mul. Fusing is the job of
``daceml_amd.transformation.fusion``; running is the job of ``daceml_amd.runtime``.
"""
import math
from typing import Dict, List, Optional, Sequence, Tuple

import torch

from . import onnx as donnx
from .sdfg import SDFG, SDFGState


class GraphBuilder:
    """Adds library nodes with their access nodes and edges; returns output array names."""
    def __init__(self, name: str, dtype: torch.dtype):
        self.sdfg = SDFG(name)
        self.state = self.sdfg.add_state("main")
        self.dtype = dtype
        self._n = 0

    def _fresh(self, prefix: str) -> str:
        self._n += 1
        return "%s_%d" % (prefix, self._n)

    def input(self, name: str, shape, dtype=None) -> str:
        self.sdfg.add_array(name, shape, dtype or self.dtype)
        return name

    def constant(self, name: str, value, dtype=None) -> str:
        t = torch.as_tensor(value, dtype=dtype or self.dtype)
        self.sdfg.add_array(name, tuple(t.shape), t.dtype)
        self.sdfg.add_constant(name, t)
        if t.numel() == 1:
            self.sdfg.constants_exact[name] = float(value)
        return name

    def output(self, array: str, name: str) -> str:
        """Rename a transient to a caller-visible output."""
        desc = self.sdfg.arrays.pop(array)
        desc.transient = False
        self.sdfg.arrays[name] = desc
        for e in self.state.edges():
            if e.data.data == array:
                e.data.data = name
        for n in self.state.nodes():
            if getattr(n, "data", None) == array:
                n.data = name
                n.label = name
        return name

    def node(self, op: str, inputs: Dict[str, str], out_shapes: Dict[str, Sequence[int]], out_dtype=None,
             label: Optional[str] = None, **attrs) -> Dict[str, str]:
        cls = donnx.get_onnx_node(op)
        node = cls(label or self._fresh(op), **attrs)
        self.state.add_node(node)
        for conn, arr in inputs.items():
            if conn not in node.in_connectors:
                node.add_in_connector(conn)
            self.state.add_edge(self.state.add_read(arr), None, node, conn, self.sdfg.make_array_memlet(arr))
        outs = {}
        for conn, shape in out_shapes.items():
            if conn not in node.out_connectors:
                node.add_out_connector(conn)
            name, _ = self.sdfg.add_transient(self._fresh(node.label + "_" + conn), shape, out_dtype or self.dtype)
            self.state.add_edge(node, conn, self.state.add_write(name), None, self.sdfg.make_array_memlet(name))
            outs[conn] = name
        return outs

    def shape(self, name: str) -> Tuple[int, ...]:
        return self.sdfg.arrays[name].shape

    # ---- exporter idioms -------------------------------------------------------------------
    def linear(self, x: str, weight: str, bias: Optional[str], prefix: str) -> str:
        """nn.Linear on an N-D input: Transpose(W) -> MatMul -> Add(bias, .)."""
        out_f, in_f = self.shape(weight)
        wt = self.node("Transpose", {"data": weight}, {"transposed": (in_f, out_f)}, label=prefix + "_wT",
                       perm=[1, 0])["transposed"]
        y = self.node("MatMul", {"A": x, "B": wt}, {"Y": self.shape(x)[:-1] + (out_f, )},
                      label=prefix + "_matmul")["Y"]
        if bias is not None:
            y = self.node("Add", {"A": bias, "B": y}, {"C": self.shape(y)}, label=prefix + "_bias")["C"]
        return y

    def layer_norm(self, x: str, gamma: str, beta: str, eps: float, prefix: str) -> str:
        """nn.LayerNorm over the last axis as exported at opset 12."""
        shp = self.shape(x)
        red = shp[:-1] + (1, )
        two = self.constant(prefix + "_two", 2.0)
        epsc = self.constant(prefix + "_eps", eps)
        mean = self.node("ReduceMean", {"data": x}, {"reduced": red}, label=prefix + "_mean", axes=[-1],
                         keepdims=1)["reduced"]
        cen = self.node("Sub", {"A": x, "B": mean}, {"C": shp}, label=prefix + "_sub")["C"]
        sq = self.node("Pow", {"X": cen, "Y": two}, {"Z": shp}, label=prefix + "_pow")["Z"]
        var = self.node("ReduceMean", {"data": sq}, {"reduced": red}, label=prefix + "_var", axes=[-1],
                        keepdims=1)["reduced"]
        ve = self.node("Add", {"A": var, "B": epsc}, {"C": red}, label=prefix + "_addeps")["C"]
        std = self.node("Sqrt", {"X": ve}, {"Y": red}, label=prefix + "_sqrt")["Y"]
        nrm = self.node("Div", {"A": cen, "B": std}, {"C": shp}, label=prefix + "_div")["C"]
        sc = self.node("Mul", {"A": nrm, "B": gamma}, {"C": shp}, label=prefix + "_scale")["C"]
        return self.node("Add", {"A": sc, "B": beta}, {"C": shp}, label=prefix + "_shift")["C"]

    def gelu(self, x: str, prefix: str) -> str:
        """Exact GELU as exported at opset 12: x * (erf(x / sqrt 2) + 1) * 0.5."""
        shp = self.shape(x)
        rt2 = self.constant(prefix + "_sqrt2", math.sqrt(2.0))
        one = self.constant(prefix + "_one", 1.0)
        half = self.constant(prefix + "_half", 0.5)
        d = self.node("Div", {"A": x, "B": rt2}, {"C": shp}, label=prefix + "_div")["C"]
        e = self.node("Erf", {"input": d}, {"output": shp}, label=prefix + "_erf")["output"]
        a = self.node("Add", {"A": e, "B": one}, {"C": shp}, label=prefix + "_add1")["C"]
        m = self.node("Mul", {"A": x, "B": a}, {"C": shp}, label=prefix + "_mulx")["C"]
        return self.node("Mul", {"A": m, "B": half}, {"C": shp}, label=prefix + "_mulhalf")["C"]

    def swish(self, x: str, prefix: str) -> str:
        shp = self.shape(x)
        s = self.node("Sigmoid", {"X": x}, {"Y": shp}, label=prefix + "_sigmoid")["Y"]
        return self.node("Mul", {"A": x, "B": s}, {"C": shp}, label=prefix + "_mul")["C"]


# weight names follow transformers' BertLayer state_dict
BERT_PARAMS = [
    ("attention.self.query", "q"), ("attention.self.key", "k"), ("attention.self.value", "v"),
    ("attention.output.dense", "o"), ("intermediate.dense", "ffn1"), ("output.dense", "ffn2"),
]


#: the arrays `bert_encoder_layer` takes besides ``x``
BERT_PARAM_NAMES = [short + suffix for _, short in BERT_PARAMS for suffix in ("_w", "_b")] + \
    ["ln1_g", "ln1_b", "ln2_g", "ln2_b"]


def bert_init_params(hidden: int, ffn: int, seed: int, bias_std: float = 0.0):
    """Synthetic parameters of one layer as fp32 NumPy arrays: weights N(0, 0.02), biases zero (or N(0, bias_std)),
    LayerNorm gamma 1 / beta 0. Deterministic in `seed`."""
    import numpy as np
    rng = np.random.default_rng(seed)
    p = {}
    for _, short in BERT_PARAMS:
        o, i = {"ffn1": (ffn, hidden), "ffn2": (hidden, ffn)}.get(short, (hidden, hidden))
        p[short + "_w"] = (rng.standard_normal((o, i)) * 0.02).astype(np.float32)
        p[short + "_b"] = (rng.standard_normal(o) * bias_std).astype(np.float32)
    for ln in ("ln1", "ln2"):
        p[ln + "_g"] = np.ones(hidden, np.float32)
        p[ln + "_b"] = np.zeros(hidden, np.float32)
    return p


def bert_encoder_layer(batch: int, seq: int, hidden: int, heads: int, ffn: int, dtype=torch.float16,
                       eps: float = 1e-12) -> SDFG:
    """One post-LN BERT encoder layer (HuggingFace ``BertLayer``; no mask, no dropout), decomposed as the
    opset-12 exporter emits it. Inputs: ``x`` and the parameters ``{q,k,v,o}_{w,b}``, ``ffn{1,2}_{w,b}``,
    ``ln{1,2}_{g,b}`` (weights stored [out, in] like nn.Linear). Output: ``y``."""
    if hidden % heads:
        raise ValueError("hidden size must be divisible by the number of heads")
    d = hidden // heads
    g = GraphBuilder("bert_encoder_layer", dtype)
    x = g.input("x", (batch, seq, hidden))
    for _, short in BERT_PARAMS:
        o, i = {"ffn1": (ffn, hidden), "ffn2": (hidden, ffn)}.get(short, (hidden, hidden))
        g.input(short + "_w", (o, i))
        g.input(short + "_b", (o, ))
    for ln in ("ln1", "ln2"):
        g.input(ln + "_g", (hidden, ))
        g.input(ln + "_b", (hidden, ))

    def heads_of(t: str, prefix: str) -> str:
        r = g.node("Reshape", {"data": t}, {"reshaped": (batch, seq, heads, d)}, label=prefix + "_split")["reshaped"]
        return g.node("Transpose", {"data": r}, {"transposed": (batch, heads, seq, d)}, label=prefix + "_heads",
                      perm=[0, 2, 1, 3])["transposed"]

    q = heads_of(g.linear(x, "q_w", "q_b", "q"), "q")
    k = heads_of(g.linear(x, "k_w", "k_b", "k"), "k")
    v = heads_of(g.linear(x, "v_w", "v_b", "v"), "v")
    kt = g.node("Transpose", {"data": k}, {"transposed": (batch, heads, d, seq)}, label="k_T",
                perm=[0, 1, 3, 2])["transposed"]
    scores = g.node("MatMul", {"A": q, "B": kt}, {"Y": (batch, heads, seq, seq)}, label="scores")["Y"]
    scale = g.constant("attn_scale", math.sqrt(d))
    scaled = g.node("Div", {"A": scores, "B": scale}, {"C": g.shape(scores)}, label="scores_scale")["C"]
    probs = g.node("Softmax", {"input": scaled}, {"output": g.shape(scaled)}, label="softmax", axis=3)["output"]
    ctx = g.node("MatMul", {"A": probs, "B": v}, {"Y": (batch, heads, seq, d)}, label="context")["Y"]
    ctx_t = g.node("Transpose", {"data": ctx}, {"transposed": (batch, seq, heads, d)}, label="context_merge",
                   perm=[0, 2, 1, 3])["transposed"]
    ctx2 = g.node("Reshape", {"data": ctx_t}, {"reshaped": (batch, seq, hidden)}, label="context_flat")["reshaped"]
    attn = g.linear(ctx2, "o_w", "o_b", "o")
    res1 = g.node("Add", {"A": attn, "B": x}, {"C": g.shape(x)}, label="residual1")["C"]
    h1 = g.layer_norm(res1, "ln1_g", "ln1_b", eps, "ln1")
    inter = g.gelu(g.linear(h1, "ffn1_w", "ffn1_b", "ffn1"), "gelu")
    out = g.linear(inter, "ffn2_w", "ffn2_b", "ffn2")
    res2 = g.node("Add", {"A": out, "B": h1}, {"C": g.shape(x)}, label="residual2")["C"]
    y = g.layer_norm(res2, "ln2_g", "ln2_b", eps, "ln2")
    g.output(y, "y")
    return g.sdfg


def mbconv_block(batch: int, cin: int, hw: int, expand: int = 6, cout: int = 48, se_reduce: int = 8, stride: int = 2,
                 dtype=torch.float32) -> SDFG:
    """EfficientNet-B0-style MBConv block with folded BatchNorm (a bias per conv): 1x1 expand + swish,
    3x3 depthwise (stride, pad 1) + swish, squeeze-excite (GlobalAveragePool, 1x1 reduce + swish, 1x1 expand +
    sigmoid, Mul), 1x1 project. Inputs ``x``, ``{expand,dw,se1,se2,proj}_{w,b}``; output ``y``."""
    g = GraphBuilder("mbconv_block", dtype)
    mid = cin * expand
    ohw = (hw + 2 - 3) // stride + 1
    x = g.input("x", (batch, cin, hw, hw))
    shapes = {"expand": (mid, cin, 1, 1), "dw": (mid, 1, 3, 3), "se1": (se_reduce, mid, 1, 1),
              "se2": (mid, se_reduce, 1, 1), "proj": (cout, mid, 1, 1)}
    for n, s in shapes.items():
        g.input(n + "_w", s)
        g.input(n + "_b", (s[0], ))

    def conv(t, name, out_shape, **attrs):
        return g.node("Conv", {"X": t, "W": name + "_w", "B": name + "_b"}, {"Y": out_shape}, label=name,
                      **attrs)["Y"]

    e = g.swish(conv(x, "expand", (batch, mid, hw, hw), kernel_shape=[1, 1]), "expand_act")
    dwc = g.swish(conv(e, "dw", (batch, mid, ohw, ohw), kernel_shape=[3, 3], strides=[stride, stride],
                       pads=[1, 1, 1, 1], group=mid), "dw_act")
    pooled = g.node("GlobalAveragePool", {"X": dwc}, {"Y": (batch, mid, 1, 1)}, label="se_pool")["Y"]
    s1 = g.swish(conv(pooled, "se1", (batch, se_reduce, 1, 1), kernel_shape=[1, 1]), "se1_act")
    s2 = conv(s1, "se2", (batch, mid, 1, 1), kernel_shape=[1, 1])
    gate = g.node("Sigmoid", {"X": s2}, {"Y": (batch, mid, 1, 1)}, label="se_gate")["Y"]
    gated = g.node("Mul", {"A": dwc, "B": gate}, {"C": g.shape(dwc)}, label="se_scale")["C"]
    y = conv(gated, "proj", (batch, cout, ohw, ohw), kernel_shape=[1, 1])
    g.output(y, "y")
    return g.sdfg
