"""CPU oracle of one BERT encoder layer, forward and backward, composed from oracle.ops.

TEST INFRASTRUCTURE ONLY (see oracle/ops.py). The forward follows the node sequence the opset-12
exporter emits for HuggingFace's ``BertLayer`` (the graph DaCeML imports in
tests/torch/test_bert_encoder.py:13-52): per-node pure expansions, one NumPy statement per reference
statement. The backward applies, node by node in reverse, the reference's registered backward
implementations (DefaultEinsumBackward / DefaultSoftmaxBackward,
daceml/autodiff/implementations/onnx_ops.py:25-138,237-275) and the closed-form reversal of the
LayerNorm / GELU / Add tasklets. Contractions go through ``np.matmul`` (BLAS), the CPU counterpart of
``set_fast_implementations`` (daceml/util/utils.py:226-229).

Pinned in tests/test_oracle.py against ``transformers`` ``BertLayer`` (forward) and ``torch.autograd``
(backward) in fp64.
"""
import math
from typing import Dict

import numpy as np

from . import ops as O

PARAM_NAMES = ["q_w", "q_b", "k_w", "k_b", "v_w", "v_b", "o_w", "o_b", "ffn1_w", "ffn1_b", "ffn2_w", "ffn2_b",
               "ln1_g", "ln1_b", "ln2_g", "ln2_b"]


def init_params(hidden: int, ffn: int, seed: int, dtype=np.float32, bias_std: float = 0.0) -> Dict[str, np.ndarray]:
    """Weights N(0, 0.02), biases zero (or N(0, bias_std)), LayerNorm gamma 1 / beta 0 — the init of
    BASELINE.json's BERT-large configs. Deterministic in `seed`."""
    rng = np.random.default_rng(seed)
    p = {}
    for name, (o, i) in (("q", (hidden, hidden)), ("k", (hidden, hidden)), ("v", (hidden, hidden)),
                         ("o", (hidden, hidden)), ("ffn1", (ffn, hidden)), ("ffn2", (hidden, ffn))):
        p[name + "_w"] = (rng.standard_normal((o, i)) * 0.02).astype(dtype)
        p[name + "_b"] = (rng.standard_normal(o) * bias_std).astype(dtype)
    for ln in ("ln1", "ln2"):
        p[ln + "_g"] = np.ones(hidden, dtype)
        p[ln + "_b"] = np.zeros(hidden, dtype)
    return p


def _linear(x, w, b):
    # Transpose(W) -> MatMul -> Add(bias, .)
    return O.add(b, np.matmul(x, O.transpose(w, [1, 0])))


def forward(x: np.ndarray, p: Dict[str, np.ndarray], heads: int, eps: float = 1e-12, keep: bool = False):
    """Returns y, or (y, saved intermediates) with keep=True."""
    bsz, seq, hidden = x.shape
    d = hidden // heads

    def split(t):  # Reshape -> Transpose(0, 2, 1, 3)
        return O.transpose(t.reshape(bsz, seq, heads, d), [0, 2, 1, 3])

    q = split(_linear(x, p["q_w"], p["q_b"]))
    k = split(_linear(x, p["k_w"], p["k_b"]))
    v = split(_linear(x, p["v_w"], p["v_b"]))
    scores = np.matmul(q, O.transpose(k, [0, 1, 3, 2]))
    scaled = O.div(scores, x.dtype.type(math.sqrt(d)))
    probs = O.softmax(scaled, axis=3)
    ctx = np.matmul(probs, v)
    ctx2 = O.transpose(ctx, [0, 2, 1, 3]).reshape(bsz, seq, hidden)
    res1 = O.add(_linear(ctx2, p["o_w"], p["o_b"]), x)
    h1, _, _ = O.layernorm_chain(res1, p["ln1_g"], p["ln1_b"], eps)
    pre = _linear(h1, p["ffn1_w"], p["ffn1_b"])
    act = O.gelu_chain(pre)
    res2 = O.add(_linear(act, p["ffn2_w"], p["ffn2_b"]), h1)
    y, _, _ = O.layernorm_chain(res2, p["ln2_g"], p["ln2_b"], eps)
    if not keep:
        return y
    return y, dict(q=q, k=k, v=v, probs=probs, ctx2=ctx2, res1=res1, h1=h1, pre=pre, act=act, res2=res2)


def backward(x: np.ndarray, p: Dict[str, np.ndarray], heads: int, dy: np.ndarray, saved: Dict[str, np.ndarray],
             eps: float = 1e-12, term_scales: bool = False) -> Dict[str, np.ndarray]:
    """Gradients w.r.t. x and every parameter (keys ``x`` and PARAM_NAMES).

    With ``term_scales`` the result also holds, under ``"terms:" + name`` for every parameter, the root of the sum of
    squares of the terms that gradient element adds up over the batch x sequence rows (``sqrt(sum_a (dout[a, j]
    inp[a, k])^2)`` for a weight): what a test needs to say how far a sum of rounded terms may be from the exact one.
    The gradients that leave the attention products (dq, dk, dv) are themselves sums over 512 keys or queries that
    cancel to a fraction of their terms; where they enter a parameter gradient they count with the root-sum-square of
    their own terms instead of their value. Not part of the reference's arithmetic."""
    bsz, seq, hidden = x.shape
    d = hidden // heads
    g: Dict[str, np.ndarray] = {}

    def linear_bwd(dout, inp, w, name, dout_scale=None):
        m = dout.reshape(-1, dout.shape[-1])
        i2 = inp.reshape(-1, inp.shape[-1])
        g[name + "_w"] = np.matmul(m.T, i2)                                   # 'aij,aik->jk'
        g[name + "_b"] = m.sum(axis=0)
        if term_scales:
            m2 = m * m if dout_scale is None else np.maximum(m * m, dout_scale.reshape(m.shape) ** 2)
            g["terms:" + name + "_w"] = np.sqrt(np.matmul(m2.T, i2 * i2))
            g["terms:" + name + "_b"] = np.sqrt(m2.sum(axis=0))
        return np.matmul(dout, w)                                             # 'aij,jk->aik'

    def layernorm_terms(dout, inp, name):
        if term_scales:
            m = dout.reshape(-1, dout.shape[-1])
            i2 = inp.reshape(-1, inp.shape[-1])
            xhat = (i2 - i2.mean(axis=1, keepdims=True)) / np.sqrt(i2.var(axis=1, keepdims=True) + eps)
            g["terms:" + name + "_g"] = np.sqrt(((m * xhat) ** 2).sum(axis=0))
            g["terms:" + name + "_b"] = np.sqrt((m * m).sum(axis=0))

    dres2, g["ln2_g"], g["ln2_b"] = O.layernorm_backward(dy, saved["res2"], p["ln2_g"], eps)
    layernorm_terms(dy, saved["res2"], "ln2")
    dact = linear_bwd(dres2, saved["act"], p["ffn2_w"], "ffn2")
    dpre = O.gelu_backward(dact, saved["pre"])
    dh1 = O.sum_variadic(dres2, linear_bwd(dpre, saved["h1"], p["ffn1_w"], "ffn1"))
    dres1, g["ln1_g"], g["ln1_b"] = O.layernorm_backward(dh1, saved["res1"], p["ln1_g"], eps)
    layernorm_terms(dh1, saved["res1"], "ln1")
    dctx2 = linear_bwd(dres1, saved["ctx2"], p["o_w"], "o")
    dctx = O.transpose(dctx2.reshape(bsz, seq, heads, d), [0, 2, 1, 3])
    dprobs = np.matmul(dctx, O.transpose(saved["v"], [0, 1, 3, 2]))
    dv = np.matmul(O.transpose(saved["probs"], [0, 1, 3, 2]), dctx)
    dscaled = O.softmax_backward(saved["probs"], dprobs, axis=3)
    dscores = dscaled / x.dtype.type(math.sqrt(d))
    dq = np.matmul(dscores, saved["k"])
    dk = np.matmul(O.transpose(dscores, [0, 1, 3, 2]), saved["q"])

    def merge(t):
        return O.transpose(t, [0, 2, 1, 3]).reshape(bsz, seq, hidden)

    sq = sk = sv = None
    if term_scales:   # root-sum-squares of the terms of dq, dk, dv
        ds2, pr2 = dscores * dscores, saved["probs"] * saved["probs"]
        sq = merge(np.sqrt(np.matmul(ds2, saved["k"] ** 2)))
        sk = merge(np.sqrt(np.matmul(O.transpose(ds2, [0, 1, 3, 2]), saved["q"] ** 2)))
        sv = merge(np.sqrt(np.matmul(O.transpose(pr2, [0, 1, 3, 2]), dctx * dctx)))
    dx_q = linear_bwd(merge(dq), x, p["q_w"], "q", sq)
    dx_k = linear_bwd(merge(dk), x, p["k_w"], "k", sk)
    dx_v = linear_bwd(merge(dv), x, p["v_w"], "v", sv)
    if term_scales:
        # the rows of the probabilities sum to one, so the value bias's gradient is the column sum of dctx itself: the
        # rounding of one dctx element reaches every dv element of its column, and the sum over them collects it whole
        g["terms:v_b"] = np.maximum(g["terms:v_b"], np.sqrt((dctx2 * dctx2).reshape(-1, hidden).sum(axis=0)))
    g["x"] = O.sum_variadic(dres1, dx_v, dx_q, dx_k)
    return g
