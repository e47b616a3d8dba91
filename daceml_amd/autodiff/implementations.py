"""Backward implementations that keep the backward pass on hand-written kernels.

Without these, the reference's generator would expand each forward node with a "pure" implementation
and differentiate the resulting tasklets symbolically (backward_pass_generator.py:425-494), which
bypasses any native forward implementation. Counterparts: ``DefaultEinsumBackward`` and
``DefaultSoftmaxBackward`` (daceml/autodiff/implementations/onnx_ops.py:54-138,237-275), the cuDNN /
ATen Conv backward (:494-733,1140-1265).
"""
from typing import List, Optional, Tuple

import torch

from .. import contraction as C
from .. import onnx as donnx
from ..sdfg import Node, contiguous_strides
from .base_abc import (AutoDiffException, BackwardContext, BackwardGroup, BackwardImplementation, BackwardResult,
                       autoregister_params)

NAME = "hip"


# ----------------------------------------------------------------------------- helpers
def _in_arr(ctx: BackwardContext, node, conn) -> Optional[str]:
    for e in ctx.forward_state.in_edges_by_connector(node, conn):
        return e.data.data
    return None


def _out_arr(ctx: BackwardContext, node, conn) -> Optional[str]:
    for e in ctx.forward_state.out_edges_by_connector(node, conn):
        return e.data.data
    return None


def connect_input_from_forward(forward_node, backward_node, ctx: BackwardContext, conn: str, as_conn: str = None):
    """Feed the array on input `conn` of the forward node to the reverse node (autodiff/utils.py)."""
    arr = _in_arr(ctx, forward_node, conn)
    _read(ctx, arr, backward_node, as_conn or conn)


def connect_output_from_forward(forward_node, backward_node, ctx: BackwardContext, conn: str, as_conn: str = None):
    """Feed a forward *output* to the reverse node — torch's save_for_backward (autodiff/utils.py:224-261)."""
    arr = _out_arr(ctx, forward_node, conn)
    _read(ctx, arr, backward_node, as_conn or conn)


def _read(ctx, arr, node, conn):
    st = ctx.backward_state
    if conn not in node.in_connectors:
        node.add_in_connector(conn)
    st.add_edge(st.add_read(arr), None, node, conn, ctx.backward_sdfg.make_array_memlet(arr))


def _write(ctx, node, conn, arr):
    st = ctx.backward_state
    if conn not in node.out_connectors:
        node.add_out_connector(conn)
    st.add_edge(node, conn, st.add_write(arr), None, ctx.backward_sdfg.make_array_memlet(arr))


def _ensure_forward_output(ctx: BackwardContext, node, conn: str, shape, dtype) -> str:
    """Make the forward node produce optional output `conn` (statistics, pre-activation) if it does not."""
    arr = _out_arr(ctx, node, conn)
    if arr is not None:
        return arr
    name, _ = ctx.forward_sdfg.add_transient("%s_%s" % (node.label, conn), shape, dtype)
    node.add_out_connector(conn)
    st = ctx.forward_state
    st.add_edge(node, conn, st.add_write(name), None, ctx.forward_sdfg.make_array_memlet(name))
    return name


def _new(ctx, op: str, label: str, **attrs):
    node = donnx.get_onnx_node(op)(label, **attrs)
    ctx.backward_state.add_node(node)
    return node


# ----------------------------------------------------------------------------- contractions
def _einsum_backward(forward_node, ctx: BackwardContext, given, required, eq: str, alpha: float, act: str,
                     bias_conn: Optional[str], residual_conn: Optional[str],
                     conns: Tuple[str, str, str] = ("Inputs__0", "Inputs__1", "Output"), group: Optional[BackwardGroup] = None,
                     skip: Tuple[str, ...] = ()):
    """`conns`: the forward node's connectors for the two operands and the result (MatMul and Gemm call them A, B, Y);
    `skip`: required connectors the caller differentiates itself, into `group`."""
    sdfg = ctx.forward_sdfg
    out = _out_arr(ctx, forward_node, conns[2])
    od = sdfg.arrays[out]
    group = group or BackwardGroup(forward_node.label + "_backward")
    req, passthrough = {}, {}
    grad_src: Optional[Tuple[Node, str]] = None   # producer of d(pre-activation) when an activation is undone
    dpre_arr = None
    if act != "none":
        if act != "gelu":
            raise AutoDiffException("no backward for activation %r" % act)
        pre = _ensure_forward_output(ctx, forward_node, "PreActivation", od.shape, od.dtype)
        gg = _new(ctx, "GeluGrad", forward_node.label + "_act_grad")
        _read(ctx, pre, gg, "X")
        group.map_input("Output_grad", gg, "dY")
        dpre_arr, _ = sdfg.add_transient("gradient_" + pre, od.shape, od.dtype)
        _write(ctx, gg, "dX", dpre_arr)

    def feed_dout(node, conn):
        if dpre_arr is not None:
            _read(ctx, dpre_arr, node, conn)
        else:
            node.add_in_connector(conn)
            group.map_input("Output_grad", node, conn)

    for conn in required:
        if conn in skip:
            continue
        if conn in conns[:2]:
            idx = conns.index(conn)
            others, rev_eq = C.reverse_equation(eq, idx)
            es = _new(ctx, "FusedEinsum", "%s_grad_%d" % (forward_node.label, idx), equation=rev_eq, alpha=alpha)
            feed_dout(es, "Inputs__0")
            connect_input_from_forward(forward_node, es, ctx, conns[others[0]], "Inputs__1")
            group.map_output(conn + "_grad", es, "Output")
            req[conn] = conn + "_grad"
        elif conn == bias_conn:
            nd = len(od.shape)
            rs = _new(ctx, "ReduceSum", forward_node.label + "_bias_grad", axes=list(range(nd - 1)), keepdims=0)
            feed_dout(rs, "data")
            group.map_output(conn + "_grad", rs, "reduced")
            req[conn] = conn + "_grad"
        elif conn == residual_conn:
            if act != "none":
                raise AutoDiffException("residual after an activation is not produced by the fusion pass")
            passthrough[conn] = "Output"
        else:
            raise AutoDiffException("unexpected input connector %r" % conn)
    return group, BackwardResult(required_grad_names=req, given_grad_names={conns[2]: "Output_grad"},
                                 passthrough=passthrough)


@autoregister_params(op="MatMul", name=NAME)
class HipMatMulBackward(BackwardImplementation):
    """The reference has no reverse node for MatMul: its generator expands the node with "pure" first
    (backward_pass_generator.py:425-494), which makes it the Einsum of pure_implementations.py:132-191, and
    differentiates that with DefaultEinsumBackward. Same here, without rewriting the forward node."""
    @staticmethod
    def backward_can_be_applied(node, state, sdfg) -> bool:
        try:
            ranks = [len(sdfg.arrays[next(iter(state.in_edges_by_connector(node, c))).data.data].shape) for c in ("A", "B")]
            return min(ranks) >= 2
        except StopIteration:
            return False

    @staticmethod
    def backward(forward_node, context, given_gradients, required_gradients):
        sdfg = context.forward_sdfg
        ra, rb = (len(sdfg.arrays[_in_arr(context, forward_node, c)].shape) for c in ("A", "B"))
        return _einsum_backward(forward_node, context, given_gradients, required_gradients, C.matmul_equation(ra, rb), 1.0,
                                "none", None, None, conns=("A", "B", "Y"))


@autoregister_params(op="Gemm", name=NAME)
class HipGemmBackward(BackwardImplementation):
    """Y = alpha op(A) op(B) + beta C (PureGemm, pure_implementations.py:380-553): A and B as for the Einsum PureGemm
    builds, with alpha folded into the two new contractions; C receives beta times the incoming gradient, summed over
    the rows where C is a vector broadcast over them (the Add's reversal plus ReverseReduce, dace_nodes.py:13-105)."""
    @staticmethod
    def backward_can_be_applied(node, state, sdfg) -> bool:
        try:
            a = sdfg.arrays[next(iter(state.in_edges_by_connector(node, "A"))).data.data]
            b = sdfg.arrays[next(iter(state.in_edges_by_connector(node, "B"))).data.data]
            return len(a.shape) == 2 and len(b.shape) == 2
        except StopIteration:
            return False

    @staticmethod
    def backward(forward_node, context, given_gradients, required_gradients):
        sdfg = context.forward_sdfg
        node = forward_node
        eq = "%s,%s->ij" % ("ki" if node.transA else "ik", "jk" if node.transB else "kj")
        group = BackwardGroup(node.label + "_backward")
        _, result = _einsum_backward(node, context, given_gradients, required_gradients, eq, float(node.alpha), "none", None,
                                     None, conns=("A", "B", "Y"), group=group, skip=("C", ))
        if "C" in required_gradients:
            beta = float(node.beta)
            yd = sdfg.arrays[_out_arr(context, node, "Y")]
            cd = sdfg.arrays[_in_arr(context, node, "C")]
            full = tuple(cd.shape) == tuple(yd.shape)
            if full and beta == 1.0:
                result.passthrough["C"] = "Y"
                return group, result
            src = None       # (node, connector) that produces the unscaled gradient; None: the incoming gradient itself
            if not full:
                if tuple(cd.shape) not in ((yd.shape[1], ), (1, yd.shape[1])):
                    raise AutoDiffException("%s: C of shape %s is not a row vector of Y %s" % (node.label, cd.shape, yd.shape))
                rs = _new(context, "ReduceSum", node.label + "_c_grad", axes=[0], keepdims=1 if len(cd.shape) == 2 else 0)
                rs.add_in_connector("data")
                group.map_input("Output_grad", rs, "data")
                rs.add_out_connector("reduced")
                src = (rs, "reduced")
            if beta != 1.0:
                mul = _new(context, "Mul", node.label + "_c_grad_scale")
                mul.add_in_connector("A")
                if src is None:
                    group.map_input("Output_grad", mul, "A")
                else:
                    tmp, _ = sdfg.add_transient(node.label + "_c_grad_unscaled", cd.shape, cd.dtype)
                    _write(context, src[0], src[1], tmp)
                    _read(context, tmp, mul, "A")
                _read(context, _scalar_constant(context, node.label + "_backward_beta", beta, cd.dtype), mul, "B")
                mul.add_out_connector("C")
                src = (mul, "C")
            group.map_output("C_grad", src[0], src[1])
            result.required_grad_names["C"] = "C_grad"
        return group, result


@autoregister_params(op="Einsum", name=NAME)
class HipEinsumBackward(BackwardImplementation):
    """DefaultEinsumBackward (onnx_ops.py:54-138): one new contraction per required input, with the
    equation of reverse_einsum_wrt_input (:25-51); they run on the same MFMA GEMM."""
    @staticmethod
    def backward_can_be_applied(node, state, sdfg) -> bool:
        try:
            ins, _ = C.parse(node.equation)
            return len(ins) == 2
        except C.NotApplicable:
            return False

    @staticmethod
    def backward(forward_node, context, given_gradients, required_gradients):
        return _einsum_backward(forward_node, context, given_gradients, required_gradients,
                                forward_node.equation.replace(" ", ""), 1.0, "none", None, None)


@autoregister_params(op="FusedEinsum", name=NAME)
class HipFusedEinsumBackward(BackwardImplementation):
    """Backward of a contraction with folded scale / bias / GELU / residual: GeluGrad on the stored
    pre-activation, a column ReduceSum for the bias, two contractions for the operands; the residual's
    gradient is the incoming gradient itself."""
    @staticmethod
    def backward_can_be_applied(node, state, sdfg) -> bool:
        return node.activation in ("none", "gelu") and not node.accumulate

    @staticmethod
    def backward(forward_node, context, given_gradients, required_gradients):
        st = context.forward_state
        conns = [e.dst_conn for e in st.in_edges(forward_node)]
        return _einsum_backward(forward_node, context, given_gradients, required_gradients,
                                forward_node.equation.replace(" ", ""), forward_node.alpha, forward_node.activation,
                                "Bias" if "Bias" in conns else None, "Residual" if "Residual" in conns else None)


# ----------------------------------------------------------------------------- softmax / layernorm
@autoregister_params(op="Softmax", name=NAME)
class HipSoftmaxBackward(BackwardImplementation):
    """DefaultSoftmaxBackward (onnx_ops.py:237-275): ``prod = y * dy``; ``sums = ReduceSum(prod, keepdims=1)``;
    ``dx = prod - y * sums``. For the last axis that is one SoftmaxGrad node (one kernel, needs the forward output); for
    any other axis the reference's own four nodes: Mul, ReduceSum, Mul, Sub. The sum runs over every axis the forward
    node made one row of (``axis`` and all behind it), as in the LogSoftmax reverse below: the reference sums over
    ``axes=[axis]`` alone, which is the same thing when the axes behind have extent 1 and otherwise is not the
    derivative of its own (coalescing) forward."""
    @staticmethod
    def backward_can_be_applied(node, state, sdfg) -> bool:
        for e in state.in_edges_by_connector(node, "input"):
            nd = len(sdfg.arrays[e.data.data].shape)
            return nd >= 1 and -nd <= node.axis < nd
        return False

    @staticmethod
    def backward(forward_node, context, given_gradients, required_gradients):
        sdfg = context.forward_sdfg
        out = _out_arr(context, forward_node, "output")
        od = sdfg.arrays[out]
        nd = len(od.shape)
        axis = forward_node.axis % nd
        if axis == nd - 1:
            sg = _new(context, "SoftmaxGrad", forward_node.label + "_backward", axis=-1)
            connect_output_from_forward(forward_node, sg, context, "output", "Y")
            return sg, BackwardResult(required_grad_names={"input": "dX"}, given_grad_names={"output": "dY"})
        label = forward_node.label + "_backward"
        group = BackwardGroup(label)
        sums_shape = tuple(1 if i >= axis else e for i, e in enumerate(od.shape))
        prod, _ = sdfg.add_transient(label + "_prod", od.shape, od.dtype)
        sums, _ = sdfg.add_transient(label + "_sums", sums_shape, od.dtype)
        scaled, _ = sdfg.add_transient(label + "_scaled", od.shape, od.dtype)
        mul1 = _new(context, "Mul", label + "_mul_dy")
        _read(context, out, mul1, "A")
        mul1.add_in_connector("B")
        group.map_input("output_grad", mul1, "B")
        _write(context, mul1, "C", prod)
        red = _new(context, "ReduceSum", label + "_sum", axes=list(range(axis, nd)), keepdims=1)
        _read(context, prod, red, "data")
        _write(context, red, "reduced", sums)
        mul2 = _new(context, "Mul", label + "_mul_sums")
        _read(context, out, mul2, "A")
        _read(context, sums, mul2, "B")
        _write(context, mul2, "C", scaled)
        sub = _new(context, "Sub", label + "_sub")
        _read(context, prod, sub, "A")
        _read(context, scaled, sub, "B")
        sub.add_out_connector("C")
        group.map_output("input_grad", sub, "C")
        return group, BackwardResult(required_grad_names={"input": "input_grad"},
                                     given_grad_names={"output": "output_grad"})


@autoregister_params(op="LogSoftmax", name=NAME)
class HipLogSoftmaxBackward(BackwardImplementation):
    """DefaultLogSoftmaxBackward (onnx_ops.py:338-373): ``dx = dy - exp(y) * ReduceSum(dy, axes=[axis], keepdims=1)``
    as the reference's own nodes - Exp, ReduceSum, Mul, Sub - with the sum over every axis the forward node made one
    row of (from ``axis`` on)."""
    @staticmethod
    def backward_can_be_applied(node, state, sdfg) -> bool:
        for e in state.in_edges_by_connector(node, "input"):
            nd = len(sdfg.arrays[e.data.data].shape)
            return nd >= 1 and -nd <= node.axis < nd
        return False

    @staticmethod
    def backward(forward_node, context, given_gradients, required_gradients):
        sdfg = context.forward_sdfg
        out = _out_arr(context, forward_node, "output")
        od = sdfg.arrays[out]
        nd = len(od.shape)
        axis = forward_node.axis % nd
        label = forward_node.label + "_backward"
        group = BackwardGroup(label)
        sums_shape = tuple(1 if i >= axis else e for i, e in enumerate(od.shape))
        probs, _ = sdfg.add_transient(label + "_exp", od.shape, od.dtype)
        sums, _ = sdfg.add_transient(label + "_sums", sums_shape, od.dtype)
        scaled, _ = sdfg.add_transient(label + "_scaled", od.shape, od.dtype)
        ex = _new(context, "Exp", label + "_exp")
        _read(context, out, ex, "input")
        _write(context, ex, "output", probs)
        red = _new(context, "ReduceSum", label + "_sum", axes=list(range(axis, nd)), keepdims=1)
        red.add_in_connector("data")
        group.map_input("output_grad", red, "data")
        _write(context, red, "reduced", sums)
        mul = _new(context, "Mul", label + "_mul")
        _read(context, probs, mul, "A")
        _read(context, sums, mul, "B")
        _write(context, mul, "C", scaled)
        sub = _new(context, "Sub", label + "_sub")
        sub.add_in_connector("A")
        group.map_input("output_grad", sub, "A")
        _read(context, scaled, sub, "B")
        sub.add_out_connector("C")
        group.map_output("input_grad", sub, "C")
        return group, BackwardResult(required_grad_names={"input": "input_grad"},
                                     given_grad_names={"output": "output_grad"})


@autoregister_params(op="FusedAttention", name=NAME)
class HipFusedAttentionBackward(BackwardImplementation):
    """One FusedAttentionGrad node; the forward node is made to emit its log-sum-exp rows, which replace the
    probability matrix that DefaultSoftmaxBackward (onnx_ops.py:237-275) would forward. An additive mask is a
    constant of the node: it is forwarded to the gradient node and gets no gradient of its own."""
    @staticmethod
    def backward_can_be_applied(node, state, sdfg) -> bool:
        return True

    @staticmethod
    def backward(forward_node, context, given_gradients, required_gradients):
        sdfg = context.forward_sdfg
        q = sdfg.arrays[_in_arr(context, forward_node, "Q")]
        pm = forward_node.q_perm
        lse_shape = tuple(1 if pm[i] < 0 else q.shape[pm[i]] for i in range(3))
        lse = _ensure_forward_output(context, forward_node, "LogSumExp", lse_shape, torch.float32)
        g = _new(context, "FusedAttentionGrad", forward_node.label + "_backward", scale=forward_node.scale,
                 q_perm=forward_node.q_perm, k_perm=forward_node.k_perm, v_perm=forward_node.v_perm,
                 o_perm=forward_node.o_perm)
        if "Mask" in required_gradients:
            raise AutoDiffException("%s: no gradient is produced for the attention mask (list the mask in the wrapper's "
                                    "inputs_to_skip, or keep the attention block unfused)" % forward_node.label)
        has_mask = any(e.dst_conn == "Mask" for e in context.forward_state.in_edges(forward_node))
        for conn in ("Q", "K", "V") + (("Mask", ) if has_mask else ()):
            connect_input_from_forward(forward_node, g, context, conn)
        connect_output_from_forward(forward_node, g, context, "Output", "O")
        _read(context, lse, g, "LogSumExp")
        req = {}
        for conn in ("Q", "K", "V"):
            if conn in required_gradients:
                req[conn] = "d" + conn
            else:  # the kernels always produce all three
                d = sdfg.arrays[_in_arr(context, forward_node, conn)]
                scratch, _ = sdfg.add_transient("%s_unused_d%s" % (forward_node.label, conn), d.shape, d.dtype)
                _write(context, g, "d" + conn, scratch)
        return g, BackwardResult(required_grad_names=req, given_grad_names={"Output": "dO"})


def _ln_backward(forward_node, ctx, x_arr, scale_conn, bias_conn, x_conns, mean_conn, rstd_conn, required):
    sdfg = ctx.forward_sdfg
    xd = sdfg.arrays[x_arr]
    rows = xd.total_size // xd.shape[-1]
    mean = _ensure_forward_output(ctx, forward_node, mean_conn, (rows, ), torch.float32)
    rstd = _ensure_forward_output(ctx, forward_node, rstd_conn, (rows, ), torch.float32)
    g = _new(ctx, "LayerNormalizationGrad", forward_node.label + "_backward", axis=-1)
    _read(ctx, x_arr, g, "X")
    connect_input_from_forward(forward_node, g, ctx, scale_conn, "scale")
    _read(ctx, mean, g, "mean")
    _read(ctx, rstd, g, "inv_std_var")
    return g, mean, rstd


@autoregister_params(op="LayerNormalization", name=NAME)
class HipLayerNormalizationBackward(BackwardImplementation):
    """Backward of the fused LayerNorm chain: one LayerNormalizationGrad node (plus the forward node's
    Mean / InvStdDev outputs, added here if the forward graph did not ask for them)."""
    @staticmethod
    def backward_can_be_applied(node, state, sdfg) -> bool:
        return True

    @staticmethod
    def backward(forward_node, context, given_gradients, required_gradients):
        x = _in_arr(context, forward_node, "X")
        g, _, _ = _ln_backward(forward_node, context, x, "Scale", "B", ["X"], "Mean", "InvStdDev", required_gradients)
        sdfg = context.forward_sdfg
        h = sdfg.arrays[x].shape[-1]
        req = {"X": "X_grad", "Scale": "scale_grad", "B": "bias_grad"}
        # the kernel always produces all three; unused ones land in scratch transients
        for conn, gconn in req.items():
            if conn not in required_gradients:
                shape = sdfg.arrays[x].shape if conn == "X" else (h, )
                dt = sdfg.arrays[x].dtype if conn == "X" else torch.float32
                name, _ = sdfg.add_transient("%s_unused_%s" % (forward_node.label, gconn), shape, dt)
                _write(context, g, gconn, name)
        return g, BackwardResult(required_grad_names={c: req[c] for c in required_gradients if c in req},
                                 given_grad_names={"Y": "Y_grad"})


@autoregister_params(op="BatchNormalization", name=NAME)
class HipBatchNormalizationBackward(BackwardImplementation):
    """Training-mode BatchNormalization: one BatchNormalizationGrad node reading X, scale and the statistics the
    forward node saved (CuDNNBatchNormBackward, daceml/autodiff/implementations/onnx_ops.py:1268-1510). The
    running statistics carry no gradient. A forward node with a fused activation hands the activation and its bias to
    the gradient node, which recomputes the normalised value."""
    @staticmethod
    def backward_can_be_applied(node, state, sdfg) -> bool:
        outs = {e.src_conn for e in state.out_edges(node)}
        return {"saved_mean", "saved_var"} <= outs

    @staticmethod
    def backward(forward_node, context, given_gradients, required_gradients):
        act = getattr(forward_node, "_activation", "none")
        g = _new(context, "BatchNormalizationGrad", forward_node.label + "_backward", epsilon=forward_node.epsilon,
                 activation=act)
        connect_input_from_forward(forward_node, g, context, "X")
        connect_input_from_forward(forward_node, g, context, "scale")
        if act != "none":
            connect_input_from_forward(forward_node, g, context, "B")
        connect_output_from_forward(forward_node, g, context, "saved_mean")
        connect_output_from_forward(forward_node, g, context, "saved_var")
        req = {"X": "dX", "scale": "dscale", "B": "dB"}
        for c in required_gradients:
            if c in req:
                g.add_out_connector(req[c])
        return g, BackwardResult(required_grad_names={c: req[c] for c in required_gradients if c in req},
                                 given_grad_names={"Y": "dY"})


# ----------------------------------------------------------------------------- elementwise
def _make_unary_backward(op: str, grad_op: str, in_conn: str, out_conn: str):
    class _B(BackwardImplementation):
        @staticmethod
        def backward(forward_node, context, given_gradients, required_gradients):
            g = _new(context, grad_op, forward_node.label + "_backward")
            connect_input_from_forward(forward_node, g, context, in_conn, "X")
            return g, BackwardResult(required_grad_names={in_conn: "dX"}, given_grad_names={out_conn: "dY"})

    _B.__name__ = "Hip%sBackward" % op
    _B.__doc__ = "dX = dY * f'(X) as one %s node." % grad_op
    return autoregister_params(op=op, name=NAME)(_B)


HipGeluBackward = _make_unary_backward("Gelu", "GeluGrad", "X", "Y")
HipSwishBackward = _make_unary_backward("Swish", "SwishGrad", "X", "Y")
HipSigmoidBackward = _make_unary_backward("Sigmoid", "SigmoidGrad", "X", "Y")
HipReluBackward = _make_unary_backward("Relu", "ReluGrad", "X", "Y")
HipTanhBackward = _make_unary_backward("Tanh", "TanhGrad", "input", "output")
HipErfBackward = _make_unary_backward("Erf", "ErfGrad", "input", "output")
HipSqrtBackward = _make_unary_backward("Sqrt", "SqrtGrad", "X", "Y")
HipExpBackward = _make_unary_backward("Exp", "ExpGrad", "input", "output")
HipLogBackward = _make_unary_backward("Log", "LogGrad", "input", "output")
HipReciprocalBackward = _make_unary_backward("Reciprocal", "ReciprocalGrad", "X", "Y")


@autoregister_params(op="Add", name=NAME)
class HipAddBackward(BackwardImplementation):
    """Add: the gradient passes through to an operand of the output's shape; a broadcast operand gets
    the gradient reduced over the broadcast (leading) dims — ReverseReduce in reverse
    (autodiff/implementations/dace_nodes.py:13-105)."""
    @staticmethod
    def backward_can_be_applied(node, state, sdfg) -> bool:
        try:
            out = next(iter(state.out_edges_by_connector(node, "C"))).data.data
            oshape = sdfg.arrays[out].shape
            for conn in ("A", "B"):
                arr = next(iter(state.in_edges_by_connector(node, conn))).data.data
                if _reduction_for(sdfg.arrays[arr].shape, oshape) is False:
                    return False
            return True
        except StopIteration:
            return False

    @staticmethod
    def backward(forward_node, context, given_gradients, required_gradients):
        sdfg = context.forward_sdfg
        oshape = sdfg.arrays[_out_arr(context, forward_node, "C")].shape
        group = BackwardGroup(forward_node.label + "_backward")
        req, passthrough = {}, {}
        for conn in required_gradients:
            shp = sdfg.arrays[_in_arr(context, forward_node, conn)].shape
            red = _reduction_for(shp, oshape)
            if red is None:
                passthrough[conn] = "C"
            else:
                rs = _new(context, "ReduceSum", "%s_%s_grad" % (forward_node.label, conn), axes=red[0], keepdims=red[1])
                rs.add_in_connector("data")
                group.map_input("C_grad", rs, "data")
                group.map_output(conn + "_grad", rs, "reduced")
                req[conn] = conn + "_grad"
        return group, BackwardResult(required_grad_names=req, given_grad_names={"C": "C_grad"},
                                     passthrough=passthrough)


def _reduction_for(shp, oshape):
    """How the gradient of a broadcast operand is summed back: (axes, keepdims), None when the shapes agree, or
    False when this form of broadcast is not covered. Covered: the operand has the output's trailing dims (bias
    vectors), or the output's rank with one adjacent run of size-1 dims (a per-channel gate [N, C, 1, 1])."""
    shp, oshape = tuple(shp), tuple(oshape)
    if shp == oshape:
        return None
    k = len(shp)
    if k < len(oshape) and oshape[len(oshape) - k:] == shp:
        return list(range(len(oshape) - k)), 0
    if k == len(oshape) and all(a == b or a == 1 for a, b in zip(shp, oshape)):
        axes = [i for i, (a, b) in enumerate(zip(shp, oshape)) if a == 1 and b != 1]
        if axes and axes == list(range(axes[0], axes[-1] + 1)):
            return axes, 1
    return False


def _broadcast_ok(node, state, sdfg) -> bool:
    try:
        out = next(iter(state.out_edges_by_connector(node, "C"))).data.data
        oshape = sdfg.arrays[out].shape
        for conn in ("A", "B"):
            arr = next(iter(state.in_edges_by_connector(node, conn))).data.data
            if _reduction_for(sdfg.arrays[arr].shape, oshape) is False:
                return False
        return True
    except StopIteration:
        return False


def _minus_one(ctx, dtype) -> str:
    sdfg = ctx.forward_sdfg
    name = "autodiff_minus_one_%s" % str(dtype).split(".")[-1]
    if name not in sdfg.arrays:
        sdfg.add_array(name, (), dtype)
        sdfg.add_constant(name, torch.tensor(-1.0, dtype=dtype))
        sdfg.constants_exact[name] = -1.0
    return name


class _ElementwiseBackward:
    """Builds the reverse of a broadcasting binary op out of the same elementwise library nodes (what the SymPy
    tasklet reversal of daceml/autodiff/backward_pass_generator.py:1284-1421 produces as generated maps, plus
    ReverseReduce, dace_nodes.py:13-105, for a broadcast operand)."""
    def __init__(self, forward_node, ctx):
        self.node, self.ctx = forward_node, ctx
        self.sdfg = ctx.forward_sdfg
        self.out = _out_arr(ctx, forward_node, "C")
        self.od = self.sdfg.arrays[self.out]
        self.group = BackwardGroup(forward_node.label + "_backward")
        self.n = 0

    def op(self, kind, a, b):
        """A binary node; an operand is an array name, or None for the given gradient. Returns (node, out conn)."""
        self.n += 1
        node = _new(self.ctx, kind, "%s_grad_%s_%d" % (self.node.label, kind.lower(), self.n))
        for conn, src in (("A", a), ("B", b)):
            node.add_in_connector(conn)
            if src is None:
                self.group.map_input("C_grad", node, conn)
            elif isinstance(src, tuple):
                tmp, _ = self.sdfg.add_transient("%s_tmp_%d" % (self.group.label, self.n), self.od.shape, self.od.dtype)
                _write(self.ctx, src[0], src[1], tmp)
                _read(self.ctx, tmp, node, conn)
            else:
                _read(self.ctx, src, node, conn)
        node.add_out_connector("C")
        return node, "C"

    def finish(self, conn, produced):
        """Route a full-shape gradient (node, connector) to input `conn`, reducing over broadcast dims if needed."""
        shp = self.sdfg.arrays[_in_arr(self.ctx, self.node, conn)].shape
        red = _reduction_for(shp, self.od.shape)
        if red is None:
            self.group.map_output(conn + "_grad", produced[0], produced[1])
            return
        self.n += 1
        tmp, _ = self.sdfg.add_transient("%s_full_%s" % (self.group.label, conn), self.od.shape, self.od.dtype)
        _write(self.ctx, produced[0], produced[1], tmp)
        rs = _new(self.ctx, "ReduceSum", "%s_%s_grad" % (self.node.label, conn), axes=red[0], keepdims=red[1])
        _read(self.ctx, tmp, rs, "data")
        self.group.map_output(conn + "_grad", rs, "reduced")


@autoregister_params(op="Mul", name=NAME)
class HipMulBackward(BackwardImplementation):
    """C = A * B: dA = dC * B, dB = dC * A (summed over broadcast dims)."""
    @staticmethod
    def backward_can_be_applied(node, state, sdfg) -> bool:
        return _broadcast_ok(node, state, sdfg)

    @staticmethod
    def backward(forward_node, context, given_gradients, required_gradients):
        b = _ElementwiseBackward(forward_node, context)
        req = {}
        for conn in required_gradients:
            other = _in_arr(context, forward_node, "B" if conn == "A" else "A")
            b.finish(conn, b.op("Mul", None, other))
            req[conn] = conn + "_grad"
        return b.group, BackwardResult(required_grad_names=req, given_grad_names={"C": "C_grad"})


@autoregister_params(op="Sub", name=NAME)
class HipSubBackward(BackwardImplementation):
    """C = A - B: dA = dC (passed through when shapes agree), dB = -dC."""
    @staticmethod
    def backward_can_be_applied(node, state, sdfg) -> bool:
        return _broadcast_ok(node, state, sdfg)

    @staticmethod
    def backward(forward_node, context, given_gradients, required_gradients):
        b = _ElementwiseBackward(forward_node, context)
        req, passthrough = {}, {}
        for conn in required_gradients:
            shp = b.sdfg.arrays[_in_arr(context, forward_node, conn)].shape
            red = _reduction_for(shp, b.od.shape)
            if conn == "A" and red is None:
                passthrough[conn] = "C"
                continue
            if conn == "A":
                rs = _new(context, "ReduceSum", "%s_A_grad" % forward_node.label, axes=red[0], keepdims=red[1])
                rs.add_in_connector("data")
                b.group.map_input("C_grad", rs, "data")
                b.group.map_output("A_grad", rs, "reduced")
            else:
                b.finish(conn, b.op("Mul", None, _minus_one(context, b.od.dtype)))
            req[conn] = conn + "_grad"
        return b.group, BackwardResult(required_grad_names=req, given_grad_names={"C": "C_grad"},
                                       passthrough=passthrough)


@autoregister_params(op="Div", name=NAME)
class HipDivBackward(BackwardImplementation):
    """C = A / B: dA = dC / B, dB = -(dC * C) / B with the forward output C."""
    @staticmethod
    def backward_can_be_applied(node, state, sdfg) -> bool:
        return _broadcast_ok(node, state, sdfg)

    @staticmethod
    def backward(forward_node, context, given_gradients, required_gradients):
        b = _ElementwiseBackward(forward_node, context)
        den = _in_arr(context, forward_node, "B")
        req = {}
        for conn in required_gradients:
            if conn == "A":
                b.finish(conn, b.op("Div", None, den))
            else:
                t = b.op("Mul", None, b.out)
                t = b.op("Div", t, den)
                b.finish(conn, b.op("Mul", t, _minus_one(context, b.od.dtype)))
            req[conn] = conn + "_grad"
        return b.group, BackwardResult(required_grad_names=req, given_grad_names={"C": "C_grad"})


@autoregister_params(op="Pow", name=NAME)
class HipPowBackward(BackwardImplementation):
    """Z = X ** p with p a scalar constant of the graph (the square of a decomposed LayerNormalization,
    pure_implementations.py:39-41): dX = dZ * p * X ** (p - 1). A gradient for the exponent is not offered."""
    @staticmethod
    def _exponent(node, state, sdfg):
        arr = next(iter(state.in_edges_by_connector(node, "Y"))).data.data
        return sdfg.constants_exact.get(arr)

    @staticmethod
    def backward_can_be_applied(node, state, sdfg) -> bool:
        try:
            x = next(iter(state.in_edges_by_connector(node, "X"))).data.data
            z = next(iter(state.out_edges_by_connector(node, "Z"))).data.data
            return (HipPowBackward._exponent(node, state, sdfg) is not None
                    and tuple(sdfg.arrays[x].shape) == tuple(sdfg.arrays[z].shape))
        except StopIteration:
            return False

    @staticmethod
    def backward(forward_node, context, given_gradients, required_gradients):
        if list(required_gradients) != ["X"]:
            raise AutoDiffException("Pow: only the base can be differentiated (node %s)" % forward_node.label)
        sdfg = context.forward_sdfg
        x = _in_arr(context, forward_node, "X")
        xd = sdfg.arrays[x]
        p = HipPowBackward._exponent(forward_node, context.forward_state, sdfg)
        group = BackwardGroup(forward_node.label + "_backward")
        label = forward_node.label

        def binary(kind, tag, a, b):
            node = _new(context, kind, "%s_grad_%s" % (label, tag))
            for conn, src in (("A", a), ("B", b)):
                node.add_in_connector(conn)
                if src is None:
                    group.map_input("Z_grad", node, conn)
                elif isinstance(src, tuple):
                    tmp, _ = sdfg.add_transient("%s_backward_%s_%s" % (label, tag, conn), xd.shape, xd.dtype)
                    _write(context, src[0], src[1], tmp)
                    _read(context, tmp, node, conn)
                else:
                    _read(context, src, node, conn)
            node.add_out_connector("C")
            return node, "C"

        if p == 2.0:
            base = x                                     # X ** 1
        else:
            pw = _new(context, "Pow", "%s_grad_pow" % label)
            _read(context, x, pw, "X")
            _read(context, _scalar_constant(context, "%s_backward_exponent" % label, p - 1.0, xd.dtype), pw, "Y")
            pw.add_out_connector("Z")
            base = (pw, "Z")
        t = binary("Mul", "times_base", None, base)
        t = binary("Mul", "times_exponent", t, _scalar_constant(context, "%s_backward_factor" % label, p, xd.dtype))
        group.map_output("X_grad", t[0], t[1])
        return group, BackwardResult(required_grad_names={"X": "X_grad"}, given_grad_names={"Z": "Z_grad"})


def _scalar_constant(ctx, name: str, value: float, dtype) -> str:
    sdfg = ctx.forward_sdfg
    if name not in sdfg.arrays:
        sdfg.add_array(name, (), dtype)
        sdfg.add_constant(name, torch.tensor(value, dtype=dtype))
        sdfg.constants_exact[name] = float(value)
    return name


def _make_reduce_backward(op: str, mean: bool):
    class _B(BackwardImplementation):
        @staticmethod
        def backward(forward_node, context, given_gradients, required_gradients):
            sdfg = context.forward_sdfg
            xd = sdfg.arrays[_in_arr(context, forward_node, "data")]
            nd = len(xd.shape)
            axes = sorted(a % nd for a in (forward_node.axes if forward_node.axes is not None else range(nd)))
            count = 1
            for a in axes:
                count *= xd.shape[a]
            kept = tuple(1 if i in axes else d for i, d in enumerate(xd.shape))
            scale = _scalar_constant(context, "%s_backward_scale" % forward_node.label, 1.0 / count if mean else 1.0,
                                     xd.dtype)
            g = _new(context, "ScaledExpand", forward_node.label + "_backward", x_shape=list(kept))
            g.add_in_connector("X")
            _read(context, scale, g, "Scale")
            g.add_out_connector("Y")
            return g, BackwardResult(required_grad_names={"data": "Y"}, given_grad_names={"reduced": "X"})

    _B.__name__ = "Hip%sBackward" % op
    _B.__doc__ = ("The gradient of %s is the given gradient broadcast back over the reduced axes%s (ReverseReduce, "
                  "daceml/autodiff/implementations/dace_nodes.py:13-105): one ScaledExpand node." %
                  (op, ", divided by their extent" if mean else ""))
    return autoregister_params(op=op, name=NAME)(_B)


HipReduceSumBackward = _make_reduce_backward("ReduceSum", False)
HipReduceMeanBackward = _make_reduce_backward("ReduceMean", True)


@autoregister_params(op="Transpose", name=NAME)
class HipTransposeBackward(BackwardImplementation):
    """The gradient of a Transpose is the Transpose of the gradient with the inverse permutation."""
    @staticmethod
    def backward(forward_node, context, given_gradients, required_gradients):
        nd = len(context.forward_sdfg.arrays[_in_arr(context, forward_node, "data")].shape)
        perm = list(reversed(range(nd))) if forward_node.perm is None else [p % nd for p in forward_node.perm]
        inverse = [perm.index(i) for i in range(nd)]
        g = _new(context, "Transpose", forward_node.label + "_backward", perm=inverse)
        g.add_in_connector("data")
        g.add_out_connector("transposed")
        return g, BackwardResult(required_grad_names={"data": "transposed"}, given_grad_names={"transposed": "data"})


@autoregister_params(op="Reshape", name=NAME)
class HipReshapeBackward(BackwardImplementation):
    """The gradient of a Reshape (pure_implementations.py:571-573, a copy into the new shape) is the incoming gradient
    copied back into the shape of the input: one more Reshape node."""
    @staticmethod
    def backward(forward_node, context, given_gradients, required_gradients):
        g = _new(context, "Reshape", forward_node.label + "_backward")
        g.add_in_connector("data")
        g.add_out_connector("reshaped")
        return g, BackwardResult(required_grad_names={"data": "reshaped"}, given_grad_names={"reshaped": "data"})


@autoregister_params(op="Pad", name=NAME)
class HipPadBackward(BackwardImplementation):
    """The gradient of a constant Pad is the incoming gradient without the padded border: one more Pad node with the
    amounts negated (and where the forward node cropped, zeros come back in)."""
    @staticmethod
    def backward_can_be_applied(node, state, sdfg) -> bool:
        return node.mode == "constant"

    @staticmethod
    def backward(forward_node, context, given_gradients, required_gradients):
        g = _new(context, "Pad", forward_node.label + "_backward", pads=[-int(p) for p in forward_node.pads], value=0.0,
                 mode="constant")
        g.add_in_connector("data")
        g.add_out_connector("output")
        return g, BackwardResult(required_grad_names={"data": "output"}, given_grad_names={"output": "data"})


@autoregister_params(op="MaxPool", name=NAME)
class HipMaxPoolBackward(BackwardImplementation):
    """DefaultMaxPoolBackward (onnx_ops.py:284-335): one MaxPoolGrad node, which reads the forward input."""
    @staticmethod
    def backward_can_be_applied(node, state, sdfg) -> bool:
        return not any(e.src_conn == "Indices" for e in state.out_edges(node))

    @staticmethod
    def backward(forward_node, context, given_gradients, required_gradients):
        g = _new(context, "MaxPoolGrad", forward_node.label + "_backward", kernel_shape=list(forward_node.kernel_shape),
                 strides=None if forward_node.strides is None else list(forward_node.strides))
        _read(context, _in_arr(context, forward_node, "X"), g, "X")
        g.add_in_connector("dY")
        g.add_out_connector("dX")
        return g, BackwardResult(required_grad_names={"X": "dX"}, given_grad_names={"Y": "dY"})


@autoregister_params(op="GlobalAveragePool", name=NAME)
class HipGlobalAveragePoolBackward(BackwardImplementation):
    """Y = mean of X over the spatial dims (img_op_implementations.py:415-417): dX = dY / (H*W), broadcast back over
    them — one ScaledExpand node."""
    @staticmethod
    def backward(forward_node, context, given_gradients, required_gradients):
        sdfg = context.forward_sdfg
        xd = sdfg.arrays[_in_arr(context, forward_node, "X")]
        count = 1
        for e in xd.shape[2:]:
            count *= e
        name = _scalar_constant(context, "%s_inv_count" % forward_node.label, 1.0 / count, xd.dtype)
        g = _new(context, "ScaledExpand", forward_node.label + "_backward")
        g.add_in_connector("X")
        _read(context, name, g, "Scale")
        g.add_out_connector("Y")
        return g, BackwardResult(required_grad_names={"X": "Y"}, given_grad_names={"Y": "X"})


# ----------------------------------------------------------------------------- convolution
@autoregister_params(op="Conv", name=NAME)
class HipConvBackward(BackwardImplementation):
    """One ConvGrad node for dX, dW, dB — the three cuDNN backward calls of onnx_ops.py:663-703. fp32; a Conv
    with a folded activation is not differentiated (un-fuse it first)."""
    @staticmethod
    def backward_can_be_applied(node, state, sdfg) -> bool:
        return getattr(node, "_activation", "none") == "none"

    @staticmethod
    def backward(forward_node, context, given_gradients, required_gradients):
        attrs = {k: getattr(forward_node, k) for k in ("auto_pad", "dilations", "group", "kernel_shape", "pads",
                                                       "strides")}
        g = _new(context, "ConvGrad", forward_node.label + "_backward", **attrs)
        connect_input_from_forward(forward_node, g, context, "X")
        connect_input_from_forward(forward_node, g, context, "W")
        names = {"X": "dX", "W": "dW", "B": "dB"}
        for c in required_gradients:
            g.add_out_connector(names[c])
        return g, BackwardResult(required_grad_names={c: names[c] for c in required_gradients},
                                 given_grad_names={"Y": "dY"})
