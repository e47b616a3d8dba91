"""Graph rewrites that turn the exporter's decomposed opset-12 graph into the nodes the HIP kernels
implement in one launch.

Modelled on the reference's pattern-replacement machinery: ``ReplacementTransformation``
(daceml/transformation/replacement.py:67-181) for the chain -> node rewrites,
``HorizontalEinsumFusion`` (daceml/transformation/einsum_fusion.py:102-151) for folding Transposes
into contractions, ``PadConvFusion`` (daceml/transformation/pad_conv_fusion.py:80-97) for folding a
neighbour into a Conv. Every rewrite keeps the graph's results equal to the composition of the pure
expansions it replaces (that composition is the oracle of the fused kernels).

    fuse_gelu                Div, Erf, Add, Mul, Mul                      -> Gelu
    fuse_layernorm           ReduceMean, Sub, Pow, ReduceMean, Add, Sqrt,
                             Div, Mul, Add                                -> LayerNormalization
    fuse_swish               Sigmoid, Mul                                 -> Swish
    lower_matmul             MatMul                                       -> Einsum (PureMatMul's lowering)
    fold_views               Transpose / Reshape around an Einsum         -> operand letters / dense views
    fuse_epilogues           Einsum, [Div|Mul const], [Add bias], [Gelu],
                             [Add residual]                               -> FusedEinsum
    fuse_skip_layernorm      Add, LayerNormalization                      -> SkipLayerNormalization
    fuse_attention           Einsum(Q,K)[*scale], Softmax, Einsum(P,V)    -> FusedAttention
    fuse_reductions          independent ReduceSum(leading axes) nodes    -> MultiReduceSum (one launch pair)
    group_einsums            independent, identically shaped FusedEinsums -> GroupedEinsum (one launch)
    fuse_pad_into_conv       Pad (zeros, spatial axes), Conv              -> Conv(pads)
    fuse_conv_activation     Conv, Swish | Sigmoid | Relu                 -> Conv(_activation)
    fuse_gate_into_conv      Mul(X, gate[n,c,1,1]), Conv 1x1              -> GatedConv (inference graphs)
"""
import math
from typing import Dict, List, Optional, Tuple

import torch

from .. import _lib
from .. import contraction as C
from .. import onnx as donnx
from ..onnx.nodes import ONNXOp
from ..sdfg import SDFG, AccessNode, Array, Edge, SDFGState, contiguous_strides


# ----------------------------------------------------------------------------- graph helpers
def _producer(state: SDFGState, array: str) -> Optional[Tuple[ONNXOp, str]]:
    for e in state.edges():
        if e.data.data == array and isinstance(e.dst, AccessNode) and not isinstance(e.src, AccessNode):
            return e.src, e.src_conn
    return None


def _consumers(state: SDFGState, array: str) -> List[Tuple[ONNXOp, str]]:
    return [(e.dst, e.dst_conn) for e in state.edges()
            if e.data.data == array and isinstance(e.src, AccessNode) and not isinstance(e.dst, AccessNode)]


def _in_array(state: SDFGState, node, conn: str) -> Optional[str]:
    for e in state.in_edges_by_connector(node, conn):
        return e.data.data
    return None


def _out_array(state: SDFGState, node, conn: str) -> Optional[str]:
    for e in state.out_edges_by_connector(node, conn):
        return e.data.data
    return None


def _is_op(node, name: str) -> bool:
    return isinstance(node, ONNXOp) and node.schema.name == name


def _internal(sdfg: SDFG, state: SDFGState, array: str, n_consumers: int = 1) -> bool:
    """A transient that only the matched pattern reads."""
    d = sdfg.arrays[array]
    return (d.transient and not getattr(d, "persistent", False) and d.view_of is None
            and len(_consumers(state, array)) == n_consumers)


def _scalar_const(sdfg: SDFG, array: Optional[str]) -> Optional[float]:
    if array is None or array not in sdfg.constants or sdfg.arrays[array].total_size != 1:
        return None
    if array in sdfg.constants_exact:
        return sdfg.constants_exact[array]
    return float(sdfg.constants[array].reshape(-1)[0])


def _remove_node(state: SDFGState, node):
    """Remove a library node together with access nodes that are left without edges."""
    neighbours = [e.src for e in state.in_edges(node)] + [e.dst for e in state.out_edges(node)]
    state.remove_node(node)
    for n in neighbours:
        if isinstance(n, AccessNode) and not state.in_edges(n) and not state.out_edges(n) and n in state.nodes():
            state.remove_node(n)


def _drop_unused_arrays(sdfg: SDFG):
    used = set()
    for st in sdfg.states():
        for e in st.edges():
            used.add(e.data.data)
    # keep bases of views that are in use
    for name in list(used):
        d = sdfg.arrays.get(name)
        while d is not None and d.view_of is not None:
            used.add(d.view_of)
            d = sdfg.arrays.get(d.view_of)
    for name in list(sdfg.arrays):
        if name not in used and sdfg.arrays[name].transient:
            del sdfg.arrays[name]
            sdfg.constants.pop(name, None)
    for name in list(sdfg.constants):
        if name not in used:
            sdfg.constants.pop(name)
            sdfg.constants_exact.pop(name, None)
            sdfg.arrays.pop(name, None)


def _add_node(sdfg: SDFG, state: SDFGState, op: str, label: str, inputs: Dict[str, str], outputs: Dict[str, str],
              **attrs) -> ONNXOp:
    node = donnx.get_onnx_node(op)(label, **attrs)
    state.add_node(node)
    for conn, arr in inputs.items():
        if conn not in node.in_connectors:
            node.add_in_connector(conn)
        state.add_edge(state.add_read(arr), None, node, conn, sdfg.make_array_memlet(arr))
    for conn, arr in outputs.items():
        if conn not in node.out_connectors:
            node.add_out_connector(conn)
        state.add_edge(node, conn, state.add_write(arr), None, sdfg.make_array_memlet(arr))
    return node


def _binary_operands(state, node) -> Tuple[str, str]:
    return _in_array(state, node, "A"), _in_array(state, node, "B")


# ----------------------------------------------------------------------------- GELU
def fuse_gelu(sdfg: SDFG) -> int:
    """x -> Div(sqrt 2) -> Erf -> Add(1) -> Mul(x, .) -> Mul(0.5)  ==>  Gelu(x)."""
    count = 0
    for state in sdfg.states():
        for erf in [n for n in state.nodes() if _is_op(n, "Erf")]:
            d_arr = _in_array(state, erf, "input")
            prod = _producer(state, d_arr)
            if prod is None or not _is_op(prod[0], "Div") or not _internal(sdfg, state, d_arr):
                continue
            div = prod[0]
            x, c = _binary_operands(state, div)
            cv = _scalar_const(sdfg, c)
            if cv is None or abs(cv - math.sqrt(2.0)) > 1e-3:
                continue
            e_arr = _out_array(state, erf, "output")
            cons = _consumers(state, e_arr)
            if len(cons) != 1 or not _is_op(cons[0][0], "Add") or not _internal(sdfg, state, e_arr):
                continue
            add = cons[0][0]
            other = [a for a in _binary_operands(state, add) if a != e_arr]
            if len(other) != 1 or _scalar_const(sdfg, other[0]) != 1.0:
                continue
            a_arr = _out_array(state, add, "C")
            cons = _consumers(state, a_arr)
            if len(cons) != 1 or not _is_op(cons[0][0], "Mul") or not _internal(sdfg, state, a_arr):
                continue
            mulx = cons[0][0]
            if set(_binary_operands(state, mulx)) != {x, a_arr}:
                continue
            m_arr = _out_array(state, mulx, "C")
            cons = _consumers(state, m_arr)
            if len(cons) != 1 or not _is_op(cons[0][0], "Mul") or not _internal(sdfg, state, m_arr):
                continue
            mulh = cons[0][0]
            other = [a for a in _binary_operands(state, mulh) if a != m_arr]
            if len(other) != 1 or _scalar_const(sdfg, other[0]) != 0.5:
                continue
            out = _out_array(state, mulh, "C")
            for n in (div, erf, add, mulx, mulh):
                _remove_node(state, n)
            _add_node(sdfg, state, "Gelu", erf.label.replace("_erf", "") + "_fused", {"X": x}, {"Y": out})
            count += 1
    _drop_unused_arrays(sdfg)
    return count


# ----------------------------------------------------------------------------- LayerNorm
def fuse_layernorm(sdfg: SDFG) -> int:
    count = 0
    for state in sdfg.states():
        for sqrt in [n for n in state.nodes() if _is_op(n, "Sqrt")]:
            m = _match_layernorm(sdfg, state, sqrt)
            if m is None:
                continue
            x, gamma, beta, eps, out, nodes = m
            for n in nodes:
                _remove_node(state, n)
            _add_node(sdfg, state, "LayerNormalization", sqrt.label.replace("_sqrt", "") + "_fused",
                      {"X": x, "Scale": gamma, "B": beta}, {"Y": out}, axis=-1, epsilon=eps)
            count += 1
    _drop_unused_arrays(sdfg)
    return count


def _match_layernorm(sdfg, state, sqrt):
    def single(arr, op):
        p = _producer(state, arr)
        return p[0] if p is not None and _is_op(p[0], op) else None

    ve = _in_array(state, sqrt, "X")
    addeps = single(ve, "Add")
    if addeps is None or not _internal(sdfg, state, ve):
        return None
    ops = _binary_operands(state, addeps)
    eps_arr = [a for a in ops if _scalar_const(sdfg, a) is not None]
    var_arr = [a for a in ops if a not in eps_arr]
    if len(eps_arr) != 1 or len(var_arr) != 1 or not _internal(sdfg, state, var_arr[0]):
        return None
    eps = _scalar_const(sdfg, eps_arr[0])
    var = single(var_arr[0], "ReduceMean")
    if var is None:
        return None
    sq_arr = _in_array(state, var, "data")
    powr = single(sq_arr, "Pow")
    if powr is None or not _internal(sdfg, state, sq_arr) or _scalar_const(sdfg, _in_array(state, powr, "Y")) != 2.0:
        return None
    cen_arr = _in_array(state, powr, "X")
    sub = single(cen_arr, "Sub")
    casts = []
    if sub is None:
        # a half-precision LayerNorm is exported with the variance computed in a wider type: Sub -> Cast -> Pow ...
        # Div -> Cast -> Mul. The fused kernel does all of its arithmetic in fp32, so the casts fold away.
        cast_in = single(cen_arr, "Cast")
        if cast_in is None:
            return None
        narrow = _in_array(state, cast_in, "input")
        sub = single(narrow, "Sub")
        if sub is None or not _internal(sdfg, state, narrow):
            return None
        casts.append(cast_in)
    if not _internal(sdfg, state, cen_arr, 2):
        return None
    x, mean_arr = _binary_operands(state, sub)
    mean = single(mean_arr, "ReduceMean")
    if mean is None or _in_array(state, mean, "data") != x or not _internal(sdfg, state, mean_arr):
        return None
    nd = len(sdfg.arrays[x].shape)
    for r in (mean, var):
        axes = [a % nd for a in (r.axes or [])]
        if axes != [nd - 1] or not r.keepdims:
            return None
    std_arr = _out_array(state, sqrt, "Y")
    cons = _consumers(state, std_arr)
    if len(cons) != 1 or not _is_op(cons[0][0], "Div") or not _internal(sdfg, state, std_arr):
        return None
    div = cons[0][0]
    if _binary_operands(state, div) != (cen_arr, std_arr):
        return None
    nrm = _out_array(state, div, "C")
    cons = _consumers(state, nrm)
    if casts:
        if len(cons) != 1 or not _is_op(cons[0][0], "Cast") or not _internal(sdfg, state, nrm):
            return None
        casts.append(cons[0][0])
        nrm = _out_array(state, cons[0][0], "output")
        if sdfg.arrays[nrm].dtype != sdfg.arrays[x].dtype:
            return None
        cons = _consumers(state, nrm)
    if len(cons) != 1 or not _is_op(cons[0][0], "Mul") or not _internal(sdfg, state, nrm):
        return None
    mul = cons[0][0]
    gamma = [a for a in _binary_operands(state, mul) if a != nrm]
    sc = _out_array(state, mul, "C")
    cons = _consumers(state, sc)
    if len(gamma) != 1 or len(cons) != 1 or not _is_op(cons[0][0], "Add") or not _internal(sdfg, state, sc):
        return None
    add = cons[0][0]
    beta = [a for a in _binary_operands(state, add) if a != sc]
    h = sdfg.arrays[x].shape[-1]
    if len(beta) != 1 or sdfg.arrays[gamma[0]].total_size != h or sdfg.arrays[beta[0]].total_size != h:
        return None
    out = _out_array(state, add, "C")
    return x, gamma[0], beta[0], eps, out, [mean, sub, powr, var, addeps, sqrt, div, mul, add] + casts


# ----------------------------------------------------------------------------- Swish
def fuse_swish(sdfg: SDFG) -> int:
    count = 0
    for state in sdfg.states():
        for sig in [n for n in state.nodes() if _is_op(n, "Sigmoid")]:
            x = _in_array(state, sig, "X")
            s = _out_array(state, sig, "Y")
            cons = _consumers(state, s)
            if len(cons) != 1 or not _is_op(cons[0][0], "Mul") or not _internal(sdfg, state, s):
                continue
            mul = cons[0][0]
            if set(_binary_operands(state, mul)) != {x, s} or sdfg.arrays[x].shape != sdfg.arrays[s].shape:
                continue
            out = _out_array(state, mul, "C")
            _remove_node(state, sig)
            _remove_node(state, mul)
            _add_node(sdfg, state, "Swish", sig.label.replace("_sigmoid", "") + "_fused", {"X": x}, {"Y": out})
            count += 1
    _drop_unused_arrays(sdfg)
    return count


def fuse_pad_into_conv(sdfg: SDFG) -> int:
    """A Pad with zeros along the spatial axes, read only by a Conv, becomes that Conv's padding (PadConvFusion,
    daceml/transformation/pad_conv_fusion.py:27-104: constant mode, fill value 0, nothing padded on the batch and
    channel axes, the padded tensor has no other reader). Two conditions more than the reference: no entry of the
    Pad is negative (a crop followed by a padded convolution is a different function), and the padding that results has
    to be the same before and after each spatial axis, which is what the convolution kernels take; a Pad
    that does not fold stays in the graph and runs on the constant-pad kernel."""
    count = 0
    for state in sdfg.states():
        for conv in [n for n in state.nodes() if _is_op(n, "Conv")]:
            xa = _in_array(state, conv, "X")
            prod = _producer(state, xa)
            if prod is None or not _is_op(prod[0], "Pad") or not _internal(sdfg, state, xa):
                continue
            pad = prod[0]
            rank = len(sdfg.arrays[xa].shape)
            nsp = rank - 2
            pads = [int(p) for p in pad.pads]
            if pad.mode != "constant" or float(pad.value) != 0.0 or rank not in (3, 4) or len(pads) != 2 * rank:
                continue
            if any(pads[i] or pads[rank + i] for i in (0, 1)) or conv.auto_pad != "NOTSET":
                continue
            if any(p < 0 for p in pads):   # a cropping Pad is not a padding of the convolution
                continue
            have = [int(p) for p in (conv.pads or [0] * (2 * nsp))]
            begin = [have[i] + pads[2 + i] for i in range(nsp)]
            end = [have[nsp + i] + pads[rank + 2 + i] for i in range(nsp)]
            if begin != end:
                continue
            src = _in_array(state, pad, "data")
            for e in list(state.in_edges_by_connector(conv, "X")):
                state.remove_edge(e)
                if isinstance(e.src, AccessNode) and not state.in_edges(e.src) and not state.out_edges(e.src):
                    state.remove_node(e.src)
            _remove_node(state, pad)
            state.add_edge(state.add_read(src), None, conv, "X", sdfg.make_array_memlet(src))
            conv.pads = begin + end
            count += 1
    if count:
        _drop_unused_arrays(sdfg)
    return count


def fuse_conv_activation(sdfg: SDFG) -> int:
    """Conv followed only by Swish / Sigmoid / Relu: the activation moves into the conv kernel."""
    names = {"Swish": "swish", "Sigmoid": "sigmoid", "Relu": "relu"}
    count = 0
    for state in sdfg.states():
        for conv in [n for n in state.nodes() if _is_op(n, "Conv")]:
            if getattr(conv, "_activation", "none") != "none":
                continue
            y = _out_array(state, conv, "Y")
            cons = _consumers(state, y)
            if len(cons) != 1 or not isinstance(cons[0][0], ONNXOp) or cons[0][0].schema.name not in names:
                continue
            if not _internal(sdfg, state, y):
                continue
            act = cons[0][0]
            out = _out_array(state, act, "Y")
            for e in state.out_edges(conv):
                state.remove_edge(e)
            _remove_node(state, act)
            for n in [n for n in state.nodes() if isinstance(n, AccessNode) and n.data == y]:
                if not state.in_edges(n) and not state.out_edges(n):
                    state.remove_node(n)
            state.add_edge(conv, "Y", state.add_write(out), None, sdfg.make_array_memlet(out))
            conv._activation = names[act.schema.name]
            count += 1
    _drop_unused_arrays(sdfg)
    return count


def fuse_batchnorm_activation(sdfg: SDFG) -> int:
    """BatchNormalization followed only by Swish / Relu: the activation moves into the normalisation kernels (forward
    and, through BatchNormalizationGrad's ``activation``, backward), which saves a pass over the tensor each way. Works
    for the inference and the training form; runs after fuse_swish."""
    names = {"Swish": "swish", "Relu": "relu"}
    count = 0
    for state in sdfg.states():
        for bn in [n for n in state.nodes() if _is_op(n, "BatchNormalization")]:
            if getattr(bn, "_activation", "none") != "none":
                continue
            y = _out_array(state, bn, "Y")
            cons = _consumers(state, y)
            if len(cons) != 1 or not isinstance(cons[0][0], ONNXOp) or cons[0][0].schema.name not in names:
                continue
            if not _internal(sdfg, state, y):
                continue
            act = cons[0][0]
            out = _out_array(state, act, "Y")
            if tuple(sdfg.arrays[out].shape) != tuple(sdfg.arrays[y].shape) or sdfg.arrays[out].dtype != sdfg.arrays[y].dtype:
                continue
            for e in [e for e in state.out_edges(bn) if e.src_conn == "Y"]:
                state.remove_edge(e)
            _remove_node(state, act)
            for n in [n for n in state.nodes() if isinstance(n, AccessNode) and n.data == y]:
                if not state.in_edges(n) and not state.out_edges(n):
                    state.remove_node(n)
            state.add_edge(bn, "Y", state.add_write(out), None, sdfg.make_array_memlet(out))
            bn._activation = names[act.schema.name]
            count += 1
    if count:
        _drop_unused_arrays(sdfg)
    return count


def fuse_gate_into_conv(sdfg: SDFG) -> int:
    """Squeeze-excite: Mul(X[n,c,h,w], gate[n,c,1,1]) read only by a pointwise Conv becomes one GatedConv, which
    saves a full read and write of X. Forward graphs only (GatedConv has no backward implementation)."""
    count = 0
    for state in sdfg.states():
        for conv in [n for n in state.nodes() if _is_op(n, "Conv")]:
            xa = _in_array(state, conv, "X")
            prod = _producer(state, xa)
            if prod is None or not _is_op(prod[0], "Mul") or not _internal(sdfg, state, xa):
                continue
            mul = prod[0]
            a, b = _in_array(state, mul, "A"), _in_array(state, mul, "B")
            xd = sdfg.arrays[xa]
            if len(xd.shape) != 4 or xd.dtype != torch.float32 or not xd.is_contiguous() \
                    or not sdfg.arrays[_out_array(state, conv, "Y")].is_contiguous():
                continue
            gate_shape = (xd.shape[0], xd.shape[1], 1, 1)
            if tuple(sdfg.arrays[b].shape) == gate_shape and tuple(sdfg.arrays[a].shape) == tuple(xd.shape):
                data, gate = a, b
            elif tuple(sdfg.arrays[a].shape) == gate_shape and tuple(sdfg.arrays[b].shape) == tuple(xd.shape):
                data, gate = b, a
            else:
                continue
            wd = sdfg.arrays[_in_array(state, conv, "W")]
            hw = xd.shape[2] * xd.shape[3]
            attrs = {k: getattr(conv, k) for k in ("auto_pad", "dilations", "group", "kernel_shape", "pads", "strides")}
            plain = (tuple(wd.shape[2:]) == (1, 1) and attrs["group"] == 1
                     and all(v == 1 for v in (attrs["strides"] or [1, 1])) and not any(attrs["pads"] or [0]))
            if not plain or xd.shape[1] % 32 or hw % 4 or hw < 128:
                continue
            ins = {"X": data, "Gate": gate, "W": _in_array(state, conv, "W")}
            bias = _in_array(state, conv, "B")
            if bias is not None:
                ins["B"] = bias
            y = _out_array(state, conv, "Y")
            act = getattr(conv, "_activation", "none")
            label = conv.label
            _remove_node(state, conv)
            _remove_node(state, mul)
            node = _add_node(sdfg, state, "GatedConv", label, ins, {"Y": y}, **attrs)
            node._activation = act
            count += 1
    if count:
        _drop_unused_arrays(sdfg)
    return count


def fuse_expand_depthwise(sdfg: SDFG) -> int:
    """Inverted-residual expansion: a pointwise Conv (+ activation) read only by a 3x3 depthwise Conv (+ activation)
    becomes one ExpandDepthwiseConv, which keeps the expanded tensor (the widest of the block) out of memory. Runs
    after fuse_conv_activation. Forward graphs only: a backward pass needs the expanded tensor."""
    count = 0
    for state in sdfg.states():
        for dw in [n for n in state.nodes() if _is_op(n, "Conv")]:
            mid = _in_array(state, dw, "X")
            prod = _producer(state, mid)
            if prod is None or not _is_op(prod[0], "Conv") or not _internal(sdfg, state, mid):
                continue
            pw = prod[0]
            if len(_consumers(state, mid)) != 1:
                continue
            x = _in_array(state, pw, "X")
            xd, md = sdfg.arrays[x], sdfg.arrays[mid]
            w1, w2 = sdfg.arrays[_in_array(state, pw, "W")], sdfg.arrays[_in_array(state, dw, "W")]
            if len(xd.shape) != 4 or any(d.dtype != torch.float32 for d in (xd, md, w1, w2)) or not xd.is_contiguous() \
                    or not sdfg.arrays[_out_array(state, dw, "Y")].is_contiguous():
                continue
            pointwise = (tuple(w1.shape[2:]) == (1, 1) and pw.group == 1 and pw.auto_pad == "NOTSET"
                         and all(v == 1 for v in (pw.strides or [1, 1])) and not any(pw.pads or [0])
                         and all(v == 1 for v in (pw.dilations or [1, 1])))
            strides = list(dw.strides or [1, 1])
            depthwise = (tuple(w2.shape) == (md.shape[1], 1, 3, 3) and dw.group == md.shape[1]
                         and dw.auto_pad == "NOTSET" and list(dw.pads or [0]) == [1, 1, 1, 1]
                         and all(v == 1 for v in (dw.dilations or [1, 1]))
                         and strides[0] == strides[1] and strides[0] in (1, 2))
            acts = (getattr(pw, "_activation", "none"), getattr(dw, "_activation", "none"))
            if not pointwise or not depthwise or acts not in EXPAND_DEPTHWISE_ACTIVATIONS:
                continue
            # the kernel's tiling: 16 input channels per step, 32 expanded channels per workgroup, and the smallest
            # row strip (three padded expanded rows of 32 channels, the 32 x (Cin + 1) weight block, the taps) must
            # fit LDS - asked of the library, which sizes the launch with the same function
            if xd.shape[1] % 16 or md.shape[1] % 32 or \
                    not _lib.load().dmlhip_conv2d_expand_depthwise_lds_bytes(xd.shape[3], xd.shape[1], strides[0]):
                continue
            ins = {"X": x, "W_pw": _in_array(state, pw, "W"), "W_dw": _in_array(state, dw, "W")}
            for conn, node in (("B_pw", pw), ("B_dw", dw)):
                bias = _in_array(state, node, "B")
                if bias is not None:
                    ins[conn] = bias
            y = _out_array(state, dw, "Y")
            label = dw.label
            _remove_node(state, dw)
            _remove_node(state, pw)
            _add_node(sdfg, state, "ExpandDepthwiseConv", label, ins, {"Y": y}, strides=strides, act_pw=acts[0],
                      act_dw=acts[1])
            count += 1
    if count:
        _drop_unused_arrays(sdfg)
    return count


# (pointwise activation, depthwise activation) pairs the fused kernel is built for
EXPAND_DEPTHWISE_ACTIVATIONS = {("swish", "swish"), ("none", "none"), ("relu", "relu"), ("swish", "none"),
                                ("none", "swish"), ("relu", "none"), ("none", "relu")}


# ----------------------------------------------------------------------------- contractions
def lower_matmul(sdfg: SDFG) -> int:
    """MatMul -> Einsum with the equation PureMatMul builds (pure_implementations.py:132-191); Gemm likewise."""
    count = 0
    for state in sdfg.states():
        for mm in [n for n in state.nodes() if _is_op(n, "MatMul")]:
            a, b = _in_array(state, mm, "A"), _in_array(state, mm, "B")
            y = _out_array(state, mm, "Y")
            ra, rb = len(sdfg.arrays[a].shape), len(sdfg.arrays[b].shape)
            if ra < 2 or rb < 2:
                continue
            eq = C.matmul_equation(ra, rb)
            _remove_node(state, mm)
            _add_node(sdfg, state, "Einsum", mm.label, {"Inputs__0": a, "Inputs__1": b}, {"Output": y}, equation=eq)
            count += 1
        # Gemm (how nn.Linear on a 2-D input is exported: transB = 1, C = the bias) -> the contraction PureGemm builds
        # (pure_implementations.py:455-553) with alpha and the bias vector folded in
        for gm in [n for n in state.nodes() if _is_op(n, "Gemm")]:
            a, b, c = _in_array(state, gm, "A"), _in_array(state, gm, "B"), _in_array(state, gm, "C")
            y = _out_array(state, gm, "Y")
            if len(sdfg.arrays[a].shape) != 2 or len(sdfg.arrays[b].shape) != 2:
                continue
            n_out = sdfg.arrays[y].shape[-1]
            if c is not None and not (float(gm.beta) == 1.0 and sdfg.arrays[c].total_size == n_out
                                      and sdfg.arrays[c].shape[-1] == n_out and sdfg.arrays[c].is_contiguous()):
                continue
            eq = "%s,%s->ij" % ("ki" if gm.transA else "ik", "jk" if gm.transB else "kj")
            ins = {"Inputs__0": a, "Inputs__1": b}
            if c is not None:
                ins["Bias"] = c
            _remove_node(state, gm)
            if c is None and float(gm.alpha) == 1.0:
                _add_node(sdfg, state, "Einsum", gm.label, ins, {"Output": y}, equation=eq)
            else:
                _add_node(sdfg, state, "FusedEinsum", gm.label, ins, {"Output": y}, equation=eq, alpha=float(gm.alpha),
                          activation="none", accumulate=0)
            count += 1
    return count


def _einsum_terms(node) -> Tuple[List[str], str]:
    ins, out = C.parse(node.equation)
    return ins, out


def _plannable(sdfg, eq: str, a: str, b: str) -> bool:
    da, db = sdfg.arrays[a], sdfg.arrays[b]
    try:
        C.plan_contraction(eq, da.shape, da.strides, db.shape, db.strides)
        return True
    except (C.NotApplicable, ValueError):
        return False


def _reshape_to_view(sdfg: SDFG, state: SDFGState, reshape) -> bool:
    """A Reshape of a dense array moves nothing: its output becomes a dense view of its input."""
    src = _in_array(state, reshape, "data")
    dst = _out_array(state, reshape, "reshaped")
    ds, dd = sdfg.arrays[src], sdfg.arrays[dst]
    if not ds.is_contiguous() or not dd.transient or ds.total_size != dd.total_size or ds.dtype != dd.dtype:
        return False
    base, off = src, 0
    while sdfg.arrays[base].view_of is not None:
        off += sdfg.arrays[base].view_offset
        base = sdfg.arrays[base].view_of
    dd.view_of, dd.view_offset = base, off
    dd.strides = contiguous_strides(dd.shape)
    _remove_node(state, reshape)
    # consumers of the view must still be ordered after the producer of the base: keep that
    # dependency visible by remembering the alias
    sdfg.arrays[dst]._alias_source = src
    return True


def fold_views(sdfg: SDFG, reshapes: bool = True) -> int:
    """Fold Transposes next to two-operand Einsums into the equation's letters, and Reshapes of dense
    arrays into views, so that head split / merge and weight transposes cost no kernel and no HBM pass.
    ``reshapes=False`` leaves the Reshape nodes alone (no aliasing descriptors are created)."""
    count = 0
    for state in sdfg.states():
        changed = True
        while changed:
            changed = False
            for es in [n for n in state.nodes() if _is_op(n, "Einsum") or _is_op(n, "FusedEinsum")]:
                terms, out_t = _einsum_terms(es)
                if len(terms) != 2:
                    continue
                arrays = [_in_array(state, es, "Inputs__0"), _in_array(state, es, "Inputs__1")]
                # ---- operands
                for i in (0, 1):
                    prod = _producer(state, arrays[i])
                    if prod is None:
                        continue
                    pnode = prod[0]
                    if _is_op(pnode, "Transpose") and sdfg.arrays[arrays[i]].transient:
                        src = _in_array(state, pnode, "data")
                        nd = len(sdfg.arrays[src].shape)
                        perm = list(reversed(range(nd))) if pnode.perm is None else [p % nd for p in pnode.perm]
                        letters = [None] * nd
                        for pos, p in enumerate(perm):
                            letters[p] = terms[i][pos]
                        new_terms = list(terms)
                        new_terms[i] = "".join(letters)
                        new_arrays = list(arrays)
                        new_arrays[i] = src
                        eq = "%s,%s->%s" % (new_terms[0], new_terms[1], out_t)
                        if not _plannable(sdfg, eq, new_arrays[0], new_arrays[1]):
                            continue
                        edge = next(iter(state.in_edges_by_connector(es, "Inputs__%d" % i)))
                        old_access = edge.src
                        state.remove_edge(edge)
                        state.add_edge(state.add_read(src), None, es, "Inputs__%d" % i, sdfg.make_array_memlet(src))
                        if not state.in_edges(old_access) and not state.out_edges(old_access):
                            state.remove_node(old_access)
                        es.equation = eq
                        if not _consumers(state, arrays[i]):
                            _remove_node(state, pnode)
                        count += 1
                        changed = True
                        break
                    if reshapes and _is_op(pnode, "Reshape") and _reshape_to_view(sdfg, state, pnode):
                        count += 1
                        changed = True
                        break
                if changed:
                    break
                # ---- result
                y = _out_array(state, es, "Output")
                cons = _consumers(state, y)
                if len(cons) == 1 and _is_op(cons[0][0], "Transpose") and _internal(sdfg, state, y) \
                        and _is_op(es, "Einsum"):
                    tr = cons[0][0]
                    nd = len(out_t)
                    perm = list(reversed(range(nd))) if tr.perm is None else [p % nd for p in tr.perm]
                    new_out = "".join(out_t[p] for p in perm)
                    eq = "%s,%s->%s" % (terms[0], terms[1], new_out)
                    if _plannable(sdfg, eq, arrays[0], arrays[1]):
                        dst = _out_array(state, tr, "transposed")
                        for e in state.out_edges(es):
                            state.remove_edge(e)
                        _remove_node(state, tr)
                        for n in [n for n in state.nodes() if isinstance(n, AccessNode) and n.data == y]:
                            if not state.in_edges(n) and not state.out_edges(n):
                                state.remove_node(n)
                        state.add_edge(es, "Output", state.add_write(dst), None, sdfg.make_array_memlet(dst))
                        es.equation = eq
                        count += 1
                        changed = True
                        break
                if reshapes and len(cons) == 1 and _is_op(cons[0][0], "Reshape") and \
                        _reshape_to_view(sdfg, state, cons[0][0]):
                    count += 1
                    changed = True
                    break
    _drop_unused_arrays(sdfg)
    return count


def fuse_epilogues(sdfg: SDFG, keep_preactivation: bool = False, activation_in_epilogue: bool = True) -> int:
    """Einsum -> [Div | Mul by a scalar constant] -> [Add bias over the last index] -> [Gelu] ->
    [Add residual of the same shape]  ==>  one FusedEinsum. With ``keep_preactivation`` the value
    before the activation stays available as the PreActivation output (training needs it). With
    ``activation_in_epilogue=False`` the chain stops in front of the Gelu, which then runs as its own
    (memory-bound, full-occupancy) kernel."""
    count = 0
    for state in sdfg.states():
        for es in [n for n in state.nodes() if _is_op(n, "Einsum")]:
            terms, out_t = _einsum_terms(es)
            if len(terms) != 2:
                continue
            a, b = _in_array(state, es, "Inputs__0"), _in_array(state, es, "Inputs__1")
            if not _plannable(sdfg, es.equation, a, b):
                continue
            cur = _out_array(state, es, "Output")
            shape = sdfg.arrays[cur].shape
            absorbed, alpha, bias, act, residual, pre = [], 1.0, None, "none", None, None

            def sole_consumer(arr):
                cons = _consumers(state, arr)
                if len(cons) == 1 and _internal(sdfg, state, arr) and isinstance(cons[0][0], ONNXOp):
                    return cons[0][0]
                return None

            nxt = sole_consumer(cur)
            # scale
            if nxt is not None and nxt.schema.name in ("Div", "Mul"):
                x, c = _binary_operands(state, nxt)
                if x != cur and nxt.schema.name == "Mul":
                    x, c = c, x
                cv = _scalar_const(sdfg, c)
                if x == cur and cv is not None and cv != 0:
                    alpha = 1.0 / cv if nxt.schema.name == "Div" else cv
                    absorbed.append(nxt)
                    cur = _out_array(state, nxt, "C")
                    nxt = sole_consumer(cur)
            # bias
            if nxt is not None and nxt.schema.name == "Add":
                other = [o for o in _binary_operands(state, nxt) if o != cur]
                if len(other) == 1:
                    od = sdfg.arrays[other[0]]
                    if (od.total_size == shape[-1] and od.shape[-1] == shape[-1] and od.is_contiguous()
                            and _producer(state, other[0]) is None):
                        bias = other[0]
                        absorbed.append(nxt)
                        cur = _out_array(state, nxt, "C")
                        nxt = sole_consumer(cur)
            # activation
            if nxt is not None and nxt.schema.name == "Gelu" and activation_in_epilogue:
                act = "gelu"
                pre = cur
                absorbed.append(nxt)
                cur = _out_array(state, nxt, "Y")
                nxt = sole_consumer(cur)
            # residual
            if nxt is not None and nxt.schema.name == "Add":
                other = [o for o in _binary_operands(state, nxt) if o != cur]
                if len(other) == 1 and sdfg.arrays[other[0]].shape == shape and sdfg.arrays[other[0]].is_contiguous() \
                        and sdfg.arrays[other[0]].dtype == sdfg.arrays[cur].dtype:
                    residual = other[0]
                    absorbed.append(nxt)
                    cur = _out_array(state, nxt, "C")
            if not absorbed:
                continue
            for n in absorbed:
                _remove_node(state, n)
            _remove_node(state, es)
            inputs = {"Inputs__0": a, "Inputs__1": b}
            if bias:
                inputs["Bias"] = bias
            if residual:
                inputs["Residual"] = residual
            outputs = {"Output": cur}
            if pre is not None and keep_preactivation:
                outputs["PreActivation"] = pre
            _add_node(sdfg, state, "FusedEinsum", es.label + "_fused", inputs, outputs, equation=es.equation,
                      alpha=alpha, activation=act)
            count += 1
    _drop_unused_arrays(sdfg)
    return count


def fuse_skip_layernorm(sdfg: SDFG) -> int:
    """Add(x, skip) -> LayerNormalization  ==>  SkipLayerNormalization (for residual Adds that did not
    end up in a GEMM epilogue)."""
    count = 0
    for state in sdfg.states():
        for ln in [n for n in state.nodes() if _is_op(n, "LayerNormalization")]:
            x = _in_array(state, ln, "X")
            prod = _producer(state, x)
            if prod is None or not _is_op(prod[0], "Add") or not _internal(sdfg, state, x):
                continue
            add = prod[0]
            p, q = _binary_operands(state, add)
            if sdfg.arrays[p].shape != sdfg.arrays[q].shape or sdfg.arrays[p].shape != sdfg.arrays[x].shape:
                continue
            if _out_array(state, ln, "Mean") or _out_array(state, ln, "InvStdDev"):
                continue
            gamma, beta = _in_array(state, ln, "Scale"), _in_array(state, ln, "B")
            out = _out_array(state, ln, "Y")
            _remove_node(state, add)
            _remove_node(state, ln)
            _add_node(sdfg, state, "SkipLayerNormalization", ln.label.replace("_fused", "") + "_skip",
                      {"input": p, "skip": q, "gamma": gamma, "beta": beta}, {"output": out}, epsilon=ln.epsilon)
            count += 1
    _drop_unused_arrays(sdfg)
    return count


def _attention_roles(eq_scores: str, eq_context: str):
    """Letters of the two contractions -> dimension roles. Returns (q_is_first, q_perm, k_perm, v_perm, o_perm) or
    None when the pair is not softmax(Q K^T) V over the last axis of the scores."""
    try:
        (t0, t1), ts = C.parse(eq_scores)
        (c0, c1), to = C.parse(eq_context)
    except (C.NotApplicable, ValueError):
        return None
    if len(set(ts)) != len(ts) or len(ts) < 2 or len(c0) != len(ts):
        return None
    key, query = ts[-1], ts[-2]
    batch = ts[:-2]
    if len(batch) > 2:
        return None
    # which scores operand holds the queries
    if query in t0 and key in t1 and query not in t1 and key not in t0:
        tq, tk, q_first = t0, t1, True
    elif query in t1 and key in t0 and query not in t0 and key not in t1:
        tq, tk, q_first = t1, t0, False
    else:
        return None
    contracted = [l for l in tq if l not in ts]
    if len(contracted) != 1 or contracted[0] not in tk or any(l not in tq or l not in tk for l in batch):
        return None
    if sorted(tq) != sorted(list(batch) + [query, contracted[0]]) or sorted(tk) != sorted(list(batch) + [key, contracted[0]]):
        return None
    hd = contracted[0]
    # context: operand 0 is the probabilities, dimension for dimension the scores
    rename = dict(zip(ts, c0))
    ckey, cquery, cbatch = rename[key], rename[query], [rename[l] for l in batch]
    if len(set(c0)) != len(c0) or ckey in to or ckey not in c1 or cquery in c1 or cquery not in to:
        return None
    head = [l for l in c1 if l != ckey and l not in cbatch]
    if len(head) != 1 or sorted(c1) != sorted(cbatch + [ckey, head[0]]) or sorted(to) != sorted(cbatch + [cquery, head[0]]):
        return None

    def perm(term, b, seq, h):
        pad = [-1] * (2 - len(b))
        return tuple(pad + [term.index(l) for l in b] + [term.index(seq), term.index(h)])

    return (q_first, perm(tq, batch, query, hd), perm(tk, batch, key, hd), perm(c1, cbatch, ckey, head[0]),
            perm(to, cbatch, cquery, head[0]))


def fuse_attention(sdfg: SDFG) -> int:
    """Einsum(Q, K) with an optional folded scale [-> Add(mask)] -> Softmax over the keys -> Einsum(P, V) becomes one
    FusedAttention node when neither the scores nor the probabilities are read by anything else. The mask (the
    padding mask of a BERT encoder, [batch, 1, 1, keys]) becomes an input of the node when the kernels can take it:
    fp16, constant along the queries; otherwise the chain stays as it is."""
    count = 0
    for state in sdfg.states():
        for sm in [n for n in state.nodes() if _is_op(n, "Softmax")]:
            x, y = _in_array(state, sm, "input"), _out_array(state, sm, "output")
            nd = len(sdfg.arrays[x].shape)
            if sm.axis % nd != nd - 1 or not _internal(sdfg, state, x) or not _internal(sdfg, state, y):
                continue
            prod = _producer(state, x)
            cons = _consumers(state, y)
            if prod is None or len(cons) != 1 or cons[0][1] != "Inputs__0":
                continue
            es, ctx = prod[0], cons[0][0]
            add, mask = None, None
            if _is_op(es, "Add"):
                # scores + mask in either operand order; the scores are the operand a contraction produces and nobody
                # else reads, the mask is whatever the other operand is
                add = es
                for sc, mc in (("A", "B"), ("B", "A")):
                    sarr = _in_array(state, add, sc)
                    p2 = _producer(state, sarr)
                    if p2 is not None and (_is_op(p2[0], "Einsum") or _is_op(p2[0], "FusedEinsum")) \
                            and _internal(sdfg, state, sarr) and tuple(sdfg.arrays[sarr].shape) == tuple(sdfg.arrays[x].shape):
                        es, mask = p2[0], _in_array(state, add, mc)
                        break
                if mask is None:
                    continue
            if not (_is_op(es, "Einsum") or _is_op(es, "FusedEinsum")) or not _is_op(ctx, "Einsum"):
                continue
            scale = 1.0
            if _is_op(es, "FusedEinsum"):
                conns = {e.dst_conn for e in state.in_edges(es)} | {e.src_conn for e in state.out_edges(es)}
                if "Bias" in conns and mask is None:
                    # a mask of a single batch entry is a vector over the keys: the bias-folding pass has taken it
                    mask = _in_array(state, es, "Bias")
                    conns.discard("Bias")
                if conns - {"Inputs__0", "Inputs__1", "Output"} or es.activation != "none" or es.accumulate:
                    continue
                scale = float(es.alpha)
            roles = _attention_roles(es.equation.replace(" ", ""), ctx.equation.replace(" ", ""))
            if roles is None:
                continue
            q_first, q_perm, k_perm, v_perm, o_perm = roles
            qa = _in_array(state, es, "Inputs__0" if q_first else "Inputs__1")
            ka = _in_array(state, es, "Inputs__1" if q_first else "Inputs__0")
            va = _in_array(state, ctx, "Inputs__1")
            oa = _out_array(state, ctx, "Output")
            ok = True
            for arr, pm in ((qa, q_perm), (ka, k_perm), (va, v_perm), (oa, o_perm)):
                d = sdfg.arrays[arr]
                if d.dtype != torch.float16 or d.shape[pm[3]] != 64 or d.strides[pm[3]] != 1 \
                        or any(d.strides[i] % 8 for i in pm[:3] if i >= 0):
                    ok = False
            if mask is not None:
                from ..onnx.op_implementations.hip_implementations import attention_mask_strides
                if attention_mask_strides(sdfg.arrays[mask], sdfg.arrays[qa], sdfg.arrays[ka], q_perm, k_perm) is None:
                    ok = False
            if not ok:
                continue
            label = ctx.label + "_attention"
            _remove_node(state, es)
            if add is not None:
                _remove_node(state, add)
            _remove_node(state, sm)
            _remove_node(state, ctx)
            ins = {"Q": qa, "K": ka, "V": va}
            if mask is not None:
                ins["Mask"] = mask
            _add_node(sdfg, state, "FusedAttention", label, ins, {"Output": oa}, scale=scale,
                      q_perm=q_perm, k_perm=k_perm, v_perm=v_perm, o_perm=o_perm)
            count += 1
    if count:
        _drop_unused_arrays(sdfg)
    return count


def fuse_bias_gradients(sdfg: SDFG) -> int:
    """A ReduceSum of dY over every axis but the last (a bias gradient; the third node DefaultEinsumBackward's
    callers emit, daceml/autodiff/implementations/onnx_ops.py:54-138) next to a contraction whose first operand is
    the same dY summed over the same indices (the weight gradient) becomes that contraction's InputSum output: the
    kernel adds up the operand tiles it multiplies anyway, and dY is not read a second time."""
    count = 0
    for state in sdfg.states():
        for red in [n for n in state.nodes() if _is_op(n, "ReduceSum")]:
            if red.keepdims:
                continue
            x, y = _in_array(state, red, "data"), _out_array(state, red, "reduced")
            xd, yd = sdfg.arrays[x], sdfg.arrays[y]
            nd = len(xd.shape)
            axes = sorted(a % nd for a in (red.axes if red.axes is not None else range(nd)))
            if nd < 2 or axes != list(range(nd - 1)) or _consumers(state, y) or xd.dtype != torch.float16 \
                    or not (xd.is_contiguous() and yd.is_contiguous()) or yd.dtype not in (torch.float16, torch.float32):
                continue
            for node, conn in _consumers(state, x):
                if not _is_op(node, "FusedEinsum") or conn != "Inputs__0" or node.activation != "none" or node.accumulate:
                    continue
                conns = {e.dst_conn for e in state.in_edges(node)} | {e.src_conn for e in state.out_edges(node)}
                if conns != {"Inputs__0", "Inputs__1", "Output"}:
                    continue
                b = sdfg.arrays[_in_array(state, node, "Inputs__1")]
                eq = node.equation.replace(" ", "")
                terms, res = eq.split("->")[0].split(","), eq.split("->")[1]
                # the last axis of dY survives into the result, every other axis of it is contracted with the other operand
                if len(terms) != 2 or terms[0][-1] not in res or any(l in res or l not in terms[1] for l in terms[0][:-1]):
                    continue
                try:
                    plan = C.plan_contraction(eq, xd.shape, xd.strides, b.shape, b.strides)
                except (C.NotApplicable, ValueError):
                    continue
                if plan.swapped or any(e != 1 for e in plan.batch) or plan.m != xd.shape[-1] \
                        or plan.m * plan.k != xd.total_size or plan.k % 64 or b.dtype != torch.float16:
                    continue
                _remove_node(state, red)
                node.add_out_connector("InputSum")
                state.add_edge(node, "InputSum", state.add_write(y), None, sdfg.make_array_memlet(y))
                count += 1
                break
    return count


def fuse_reductions(sdfg: SDFG, max_group: int = 8) -> int:
    """Horizontal fusion (cf. HorizontalEinsumFusion, daceml/transformation/einsum_fusion.py:102-151) of ReduceSum
    nodes that sum over every axis but the last with keepdims=0 and whose results nobody in the state reads
    (bias gradients): each is a latency-bound pair of tiny launches on its own. Returns the number of nodes
    that were merged away."""
    merged = 0
    for state in sdfg.states():
        cands = {}
        for n in state.nodes():
            if not _is_op(n, "ReduceSum") or n.keepdims:
                continue
            x, y = _in_array(state, n, "data"), _out_array(state, n, "reduced")
            xd, yd = sdfg.arrays[x], sdfg.arrays[y]
            nd = len(xd.shape)
            axes = sorted(a % nd for a in (n.axes if n.axes is not None else range(nd)))
            if nd < 2 or axes != list(range(nd - 1)) or _consumers(state, y):
                continue
            vec = 8 if xd.dtype == torch.float16 else 4
            if not (xd.is_contiguous() and yd.is_contiguous()) or xd.shape[-1] % vec or xd.dtype not in (torch.float16, torch.float32):
                continue
            cands.setdefault((xd.dtype, yd.dtype), []).append((n, x, y))
        for group in cands.values():
            for i in range(0, len(group), max_group):
                part = group[i:i + max_group]
                if len(part) < 2:
                    continue
                ins = {"data__%d" % j: x for j, (_, x, _) in enumerate(part)}
                outs = {"reduced__%d" % j: y for j, (_, _, y) in enumerate(part)}
                for n, _, _ in part:
                    _remove_node(state, n)
                _add_node(sdfg, state, "MultiReduceSum", "multi_" + part[0][0].label, ins, outs)
                merged += len(part) - 1
    return merged


def _reachable(sdfg: SDFG, state: SDFGState, src) -> set:
    """Nodes reachable from `src` along the state's edges."""
    succ = {}
    for e in state.edges():
        succ.setdefault(e.src, []).append(e.dst)

    def root(name):
        while sdfg.arrays[name].view_of is not None:
            name = sdfg.arrays[name].view_of
        return name

    # access nodes of one buffer are distinct objects per use, and views alias their base: join them by root array
    by_array = {}
    for n in state.nodes():
        if isinstance(n, AccessNode):
            by_array.setdefault(root(n.data), []).append(n)
    seen, stack = set(), [src]
    while stack:
        n = stack.pop()
        nxt = list(succ.get(n, []))
        if isinstance(n, AccessNode):
            nxt += [m for m in by_array[root(n.data)] if m is not n]
        for m in nxt:
            if m not in seen:
                seen.add(m)
                stack.append(m)
    return seen


def group_einsums(sdfg: SDFG, max_group: int = 4) -> int:
    """Horizontal fusion of contractions (cf. HorizontalEinsumFusion, daceml/transformation/einsum_fusion.py:102-151):
    FusedEinsum nodes with the same equation, scale, operand shapes / strides / types (optionally a bias each, no
    residual, activation or accumulation) and no data dependence on each other become one GroupedEinsum — the
    Q/K/V projections of an attention block, and in the backward pass their input and weight gradients. Works on
    every state, so it is run after autodiff. Returns the number of nodes merged away."""
    merged = 0
    for state in sdfg.states():
        buckets = {}
        for n in state.nodes():
            if not _is_op(n, "FusedEinsum") or n.activation != "none" or n.accumulate:
                continue
            conns = {e.dst_conn for e in state.in_edges(n)} | {e.src_conn for e in state.out_edges(n)}
            if conns - {"Inputs__0", "Inputs__1", "Bias", "Output", "InputSum"} \
                    or not {"Inputs__0", "Inputs__1", "Output"} <= conns:
                continue
            a = sdfg.arrays[_in_array(state, n, "Inputs__0")]
            b = sdfg.arrays[_in_array(state, n, "Inputs__1")]
            o = sdfg.arrays[_out_array(state, n, "Output")]
            if a.dtype != torch.float16 or b.dtype != torch.float16 or not o.is_contiguous():
                continue
            bias = _in_array(state, n, "Bias")
            isum = _out_array(state, n, "InputSum")
            key = (n.equation.replace(" ", ""), float(n.alpha), tuple(a.shape), tuple(a.strides), tuple(b.shape),
                   tuple(b.strides), tuple(o.shape), o.dtype, None if bias is None else sdfg.arrays[bias].dtype,
                   None if isum is None else sdfg.arrays[isum].dtype)
            buckets.setdefault(key, []).append(n)
        for key, nodes in buckets.items():
            if len(nodes) < 2:
                continue
            nodes.sort(key=lambda n: n.label)   # the result must not depend on the order the state lists its nodes in
            try:
                plan = C.plan_contraction(key[0], key[2], key[3], key[4], key[5])
            except (C.NotApplicable, ValueError):
                continue
            if plan.batch[0] != 1:
                continue
            # greedy grouping of mutually independent nodes
            reach = {n: _reachable(sdfg, state, n) for n in nodes}
            groups: List[List[ONNXOp]] = []
            for n in nodes:
                for grp in groups:
                    if len(grp) < max_group and all(n not in reach[m] and m not in reach[n] for m in grp):
                        grp.append(n)
                        break
                else:
                    groups.append([n])
            for grp in groups:
                if len(grp) < 2:
                    continue
                ins, outs = {}, {}
                for i, n in enumerate(grp):
                    ins["A__%d" % i] = _in_array(state, n, "Inputs__0")
                    ins["B__%d" % i] = _in_array(state, n, "Inputs__1")
                    bias = _in_array(state, n, "Bias")
                    if bias is not None:
                        ins["Bias__%d" % i] = bias
                    outs["Output__%d" % i] = _out_array(state, n, "Output")
                    isum = _out_array(state, n, "InputSum")
                    if isum is not None:
                        outs["InputSum__%d" % i] = isum
                label = "grouped_" + "_".join(n.label.replace("_matmul_fused", "") for n in grp)
                for n in grp:
                    _remove_node(state, n)
                _add_node(sdfg, state, "GroupedEinsum", label, ins, outs, equation=key[0], alpha=key[1])
                merged += len(grp) - 1
    return merged


def fuse_einsum_sums(sdfg: SDFG, max_group: int = 4) -> int:
    """Gradient accumulation folded into the contractions that feed it. Autodiff sums the contributions of an
    array's consumers with an ONNXSum (daceml/autodiff/backward_pass_generator.py:715-752); when contributions are
    plain contractions of one shape (the input gradients of the Q/K/V projections) they become one EinsumSum —
    operand pairs concatenated along K, partial products never written — and a single remaining summand rides
    along as the residual of the epilogue. A Sum of one contraction and one other array becomes that contraction
    with a Residual. Returns the number of Sum operands that no longer pass through memory."""
    saved = 0
    for state in sdfg.states():
        for sm in [n for n in state.nodes() if _is_op(n, "Sum")]:
            arrays = [e.data.data for e in state.in_edges(sm)]
            out = _out_array(state, sm, "sum")
            od = sdfg.arrays[out]
            if od.dtype != torch.float16 or not od.is_contiguous() or len(set(arrays)) != len(arrays):
                continue
            viewed = {d.view_of for d in sdfg.arrays.values() if d.view_of is not None}
            buckets, producer_of = {}, {}
            for arr in arrays:
                prod = _producer(state, arr)
                d = sdfg.arrays[arr]
                if prod is None or not _is_op(prod[0], "FusedEinsum") or not _internal(sdfg, state, arr) or arr in viewed \
                        or (d.shape, d.strides, d.dtype) != (od.shape, od.strides, od.dtype):
                    continue
                n = prod[0]
                conns = {e.dst_conn for e in state.in_edges(n)} | {e.src_conn for e in state.out_edges(n)}
                if conns != {"Inputs__0", "Inputs__1", "Output"} or n.activation != "none" or n.accumulate:
                    continue
                a = sdfg.arrays[_in_array(state, n, "Inputs__0")]
                b = sdfg.arrays[_in_array(state, n, "Inputs__1")]
                if a.dtype != torch.float16 or b.dtype != torch.float16:
                    continue
                key = (n.equation.replace(" ", ""), float(n.alpha), tuple(a.shape), tuple(a.strides), tuple(b.shape),
                       tuple(b.strides))
                buckets.setdefault(key, []).append(arr)
                producer_of[arr] = n
            if not buckets:
                continue
            key, grp = max(buckets.items(), key=lambda kv: len(kv[1]))
            grp = sorted(grp, key=lambda arr: producer_of[arr].label)[:max_group]
            others = [arr for arr in arrays if arr not in grp]
            residual = others[0] if len(others) == 1 else None
            if residual is not None:
                rd = sdfg.arrays[residual]
                if (rd.shape, rd.strides, rd.dtype) != (od.shape, od.strides, od.dtype):
                    residual = None
            if len(grp) == 1:
                if residual is None:
                    continue
                # the contraction writes the sum itself
                n = producer_of[grp[0]]
                ins = {"Inputs__0": _in_array(state, n, "Inputs__0"), "Inputs__1": _in_array(state, n, "Inputs__1"),
                       "Residual": residual}
                attrs = dict(equation=n.equation, alpha=n.alpha, activation="none", accumulate=0)
                label = n.label
                _remove_node(state, sm)
                _remove_node(state, n)
                _add_node(sdfg, state, "FusedEinsum", label, ins, {"Output": out}, **attrs)
                saved += 2
                continue
            try:
                C.plan_contraction(key[0], key[2], key[3], key[4], key[5])
            except (C.NotApplicable, ValueError):
                continue
            ins = {}
            for i, arr in enumerate(grp):
                n = producer_of[arr]
                ins["A__%d" % i] = _in_array(state, n, "Inputs__0")
                ins["B__%d" % i] = _in_array(state, n, "Inputs__1")
            label = "sum_" + "_".join(producer_of[arr].label.replace("_matmul_fused", "") for arr in grp)
            sum_label = sm.label
            rest = [arr for arr in others if arr != residual] if residual is not None else others
            _remove_node(state, sm)
            for arr in grp:
                _remove_node(state, producer_of[arr])
            if residual is not None:
                ins["Residual"] = residual
            if rest:
                target, _ = sdfg.add_transient(label + "_out", od.shape, od.dtype)
            else:
                target = out
            _add_node(sdfg, state, "EinsumSum", label, ins, {"Output": target}, equation=key[0], alpha=key[1])
            if rest:
                _add_node(sdfg, state, "Sum", sum_label, {"data_0__%d" % i: arr for i, arr in enumerate([target] + rest)},
                          {"sum": out})
            saved += len(grp) + (1 if residual is not None else 0) - (1 if rest else 0)
    if saved:
        _drop_unused_arrays(sdfg)
    return saved


def fuse_mul_reduce(sdfg: SDFG) -> int:
    """Mul of two equal-shaped arrays whose product only a ReduceSum over the trailing axes reads becomes one
    MulReduceSum (a dot product per row): the product tensor disappears. This is what the reversal of a broadcast
    multiplication leaves for the broadcast operand, e.g. the gradient of a squeeze-excite gate."""
    count = 0
    for state in sdfg.states():
        for red in [n for n in state.nodes() if _is_op(n, "ReduceSum")]:
            data = _in_array(state, red, "data")
            prod = _producer(state, data)
            if prod is None or not _is_op(prod[0], "Mul") or not _internal(sdfg, state, data):
                continue
            mul = prod[0]
            a, b = _in_array(state, mul, "A"), _in_array(state, mul, "B")
            da, db, dd = sdfg.arrays[a], sdfg.arrays[b], sdfg.arrays[data]
            if not (tuple(da.shape) == tuple(db.shape) == tuple(dd.shape) and da.dtype == db.dtype == dd.dtype):
                continue
            if not (da.is_contiguous() and db.is_contiguous()):
                continue
            nd = len(dd.shape)
            axes = sorted(set(range(nd) if red.axes is None else [x % nd for x in red.axes]))
            if not axes or axes != list(range(axes[0], nd)):          # the trailing axes, all of them
                continue
            out = _out_array(state, red, "reduced")
            if sdfg.arrays[out].dtype != dd.dtype:
                continue
            label = red.label
            keep = red.keepdims
            _remove_node(state, red)
            _remove_node(state, mul)
            _add_node(sdfg, state, "MulReduceSum", label, {"A": a, "B": b}, {"reduced": out}, axes=axes, keepdims=keep)
            count += 1
    if count:
        _drop_unused_arrays(sdfg)
    return count


def _per_row_of(full, per_row) -> bool:
    """`per_row` is `full` with a (non-empty) run of trailing axes collapsed to 1."""
    full, per_row = tuple(full), tuple(per_row)
    if len(full) != len(per_row) or full == per_row:
        return False
    k = len(full)
    while k > 0 and per_row[k - 1] == 1:
        k -= 1
    return per_row[:k] == full[:k]


def fuse_row_affine(sdfg: SDFG) -> int:
    """A gradient-accumulation Sum of exactly Mul(A, S) and ScaledExpand(T, Scale), with S and T holding one value per
    row of A, becomes one RowAffine node: the two summands are never written. This is the meeting point of the two
    gradient paths of a squeeze-excite block (through the gate multiplication and through the average pool)."""
    count = 0
    for state in sdfg.states():
        for add in [n for n in state.nodes() if _is_op(n, "Sum")]:
            ins = [e.data.data for e in state.in_edges(add)]
            if len(ins) != 2:
                continue
            prods = [_producer(state, a) for a in ins]
            if any(p is None for p in prods) or not all(_internal(sdfg, state, a) for a in ins):
                continue
            kinds = [p[0].schema.name if isinstance(p[0], ONNXOp) else "" for p in prods]
            if sorted(kinds) != ["Mul", "ScaledExpand"]:
                continue
            mul = prods[kinds.index("Mul")][0]
            exp = prods[kinds.index("ScaledExpand")][0]
            out = _out_array(state, add, "sum")
            oshape = tuple(sdfg.arrays[out].shape)
            ma, mb = _in_array(state, mul, "A"), _in_array(state, mul, "B")
            if tuple(sdfg.arrays[ma].shape) == oshape and _per_row_of(oshape, sdfg.arrays[mb].shape):
                dense, factor = ma, mb
            elif tuple(sdfg.arrays[mb].shape) == oshape and _per_row_of(oshape, sdfg.arrays[ma].shape):
                dense, factor = mb, ma
            else:
                continue
            t = _in_array(state, exp, "X")
            kept = tuple(exp.x_shape) if exp.x_shape is not None else tuple(sdfg.arrays[t].shape)
            if kept != tuple(sdfg.arrays[factor].shape) or not all(
                    sdfg.arrays[x].is_contiguous() for x in (dense, factor, t)):
                continue
            if len({sdfg.arrays[x].dtype for x in (dense, factor, t, out)}) != 1:
                continue
            new_ins = {"A": dense, "S": factor, "T": t, "Scale": _in_array(state, exp, "Scale")}
            label = add.label
            _remove_node(state, add)
            _remove_node(state, mul)
            _remove_node(state, exp)
            _add_node(sdfg, state, "RowAffine", label, new_ins, {"Y": out})
            count += 1
    if count:
        _drop_unused_arrays(sdfg)
    return count


def optimize_backward(sdfg: SDFG) -> Dict[str, int]:
    """Rewrites for the state(s) autodiff added — what a ``post_autodiff_hooks`` entry of the reference's module
    wrapper would run (daceml/torch/module.py:46-365)."""
    stats = {"bias_gradients": fuse_bias_gradients(sdfg)}
    stats["mul_reductions"] = fuse_mul_reduce(sdfg)    # before fuse_reductions: these sums stop being plain ReduceSums
    stats["row_affine"] = fuse_row_affine(sdfg)
    stats["reductions"] = fuse_reductions(sdfg)
    stats["einsum_sums"] = fuse_einsum_sums(sdfg)      # before grouping: a summed group needs no separate outputs
    stats["grouped_einsums"] = group_einsums(sdfg)
    return stats


def auto_optimize(sdfg: SDFG, training: bool = False, attention: bool = True,
                  gelu_epilogue: bool = False, views: bool = True) -> Dict[str, int]:
    """The pass pipeline, in dependency order (cf. daceml.util.utils.auto_optimize,
    daceml/util/utils.py:205-235). Returns how often each rewrite fired.

    ``gelu_epilogue``: fold a Gelu that follows a contraction into the GEMM epilogue. Off by default: measured on
    MI355X (BERT-large FFN1, 4096 x 4096 x 1024) the fused epilogue costs 77 - 83 us against 47 us for the plain
    product plus 17 us for a separate Gelu kernel — the activation's arithmetic runs while the matrix pipe of the
    same wavefronts idles, whereas the separate kernel is a full-occupancy streaming pass."""
    stats = {}
    stats["gelu"] = fuse_gelu(sdfg)
    stats["layernorm"] = fuse_layernorm(sdfg)
    stats["swish"] = fuse_swish(sdfg)
    stats["pad_into_conv"] = fuse_pad_into_conv(sdfg)
    # a Conv with a folded activation, GatedConv and SkipLayerNormalization have no backward implementation: graphs that
    # will be differentiated keep those nodes apart
    stats["conv_activation"] = 0 if training else fuse_conv_activation(sdfg)
    stats["batchnorm_activation"] = fuse_batchnorm_activation(sdfg)
    stats["gated_conv"] = 0 if training else fuse_gate_into_conv(sdfg)
    stats["expand_depthwise"] = 0 if training else fuse_expand_depthwise(sdfg)
    stats["matmul_to_einsum"] = lower_matmul(sdfg)
    # views=False folds Transposes into the equations of the contractions next to them but keeps Reshape nodes: for
    # callers that hand the graph to a host with a view mechanism of its own (daceml_amd.dace_plugin.fuse_library_nodes)
    stats["views"] = fold_views(sdfg, reshapes=views)
    stats["epilogues"] = fuse_epilogues(sdfg, keep_preactivation=training, activation_in_epilogue=gelu_epilogue)
    stats["skip_layernorm"] = 0 if training else fuse_skip_layernorm(sdfg)
    stats["attention"] = fuse_attention(sdfg) if attention else 0
    # with a backward pass to come, grouping waits until after autodiff (optimize_backward): the backward
    # implementations differentiate the single contractions
    stats["grouped_einsums"] = 0 if training else group_einsums(sdfg)
    return stats
