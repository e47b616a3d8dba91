"""ONNX library nodes: one ``ONNX<Op>`` class per operator on the hot path.

Mirror of the public surface of daceml/onnx/nodes/onnx_op.py: node classes with ONNX connector
names (variadic ones as ``<name>__<i>``, daceml/onnx/nodes/node_utils.py:4-22), attributes as
properties, ``validate()`` (onnx_op.py:213-431, reduced to the checks that matter here: required
connectors, variadic numbering, one floating type per node), and a per-class implementation
registry with three selection levels — ``node.implementation``, ``ONNX<Op>.default_implementation``
and the package-wide ``daceml_amd.onnx.default_implementation`` (onnx_op.py:639-704,
daceml/onnx/__init__.py:8-9).

The reference generates its classes from the opset-12 schema database of the ``onnx`` package
(onnx_op.py:494-512); that package is not available here, so the schemas of the operators on the path
are written out below. LayerNormalization, SkipLayerNormalization, Gelu and BiasGelu do not exist in
opset 12: they are the targets of the fusion pass (daceml_amd/transformation/fusion.py) that replaces
the exporter's decomposed chains.
"""
import dataclasses
import logging
from typing import Dict, List, Optional, Tuple

import torch

from ..sdfg import SDFG, Node, SDFGState, FLOAT_DTYPES

log = logging.getLogger(__name__)


class NotApplicable(RuntimeError):
    """Raised when the selected implementation refuses a node (there is no ONNX Runtime fallback)."""


def parse_variadic_param(param: str) -> Tuple[str, int]:
    """daceml/onnx/nodes/node_utils.py:4-22."""
    split = param.split('__')
    if len(split) != 2:
        raise ValueError("Unable to parse variadic parameter '{}'".format(param))
    name, number = split
    if not number.isdigit():
        raise ValueError("Variadic parameters must be numbered, got: '{}'".format(param))
    if number[0] == '0' and len(number) > 1:
        raise ValueError("Variadic parameters must not be numbered with leading zeroes, got: '{}'".format(number))
    return name, int(number)


@dataclasses.dataclass
class ONNXParameter:
    name: str
    kind: str = "single"  # single | optional | variadic | variadic?


@dataclasses.dataclass
class ONNXSchema:
    name: str
    inputs: List[ONNXParameter]
    outputs: List[ONNXParameter]
    attributes: Dict[str, object]          # name -> default (REQUIRED for required attributes)
    since_version: int = 12

    def non_variadic_inputs(self):
        return [p.name for p in self.inputs if not p.kind.startswith("variadic")]

    def variadic_inputs(self):
        return [p.name for p in self.inputs if p.kind.startswith("variadic")]

    def non_variadic_outputs(self):
        return [p.name for p in self.outputs if not p.kind.startswith("variadic")]

    def variadic_outputs(self):
        return [p.name for p in self.outputs if p.kind.startswith("variadic")]


REQUIRED = object()


def _p(spec: str) -> List[ONNXParameter]:
    out = []
    for tok in spec.split():
        if tok.endswith("*?"):
            out.append(ONNXParameter(tok[:-2], "variadic?"))   # variadic, and allowed to be absent altogether
        elif tok.endswith("?"):
            out.append(ONNXParameter(tok[:-1], "optional"))
        elif tok.endswith("*"):
            out.append(ONNXParameter(tok[:-1], "variadic"))
        else:
            out.append(ONNXParameter(tok))
    return out


def _schema(name, ins, outs, since=12, **attrs):
    return ONNXSchema(name, _p(ins), _p(outs), attrs, since)


# connector and attribute names as used by the reference's pure implementations
# (pure_implementations.py / img_op_implementations.py parameter names)
SCHEMAS = [
    _schema("MatMul", "A B", "Y"),
    _schema("Einsum", "Inputs*", "Output", equation=REQUIRED),
    _schema("Gemm", "A B C?", "Y", alpha=1.0, beta=1.0, transA=0, transB=0),
    _schema("Softmax", "input", "output", axis=1),
    _schema("LogSoftmax", "input", "output", axis=1),
    _schema("Add", "A B", "C"), _schema("Sub", "A B", "C"), _schema("Mul", "A B", "C"), _schema("Div", "A B", "C"),
    _schema("Pow", "X Y", "Z"),
    _schema("Sqrt", "X", "Y"), _schema("Relu", "X", "Y"), _schema("Sigmoid", "X", "Y"),
    _schema("Reciprocal", "X", "Y"),
    _schema("Erf", "input", "output"), _schema("Exp", "input", "output"), _schema("Log", "input", "output"),
    _schema("Tanh", "input", "output"), _schema("Identity", "input", "output"),
    _schema("Sum", "data_0*", "sum"),
    _schema("ReduceMean", "data", "reduced", axes=None, keepdims=1),
    _schema("ReduceSum", "data", "reduced", axes=None, keepdims=1),
    _schema("ReduceMax", "data", "reduced", axes=None, keepdims=1),
    _schema("ReduceMin", "data", "reduced", axes=None, keepdims=1),
    _schema("Transpose", "data", "transposed", perm=None),
    _schema("Reshape", "data shape?", "reshaped"),
    _schema("Cast", "input", "output", to=REQUIRED),
    _schema("Conv", "X W B?", "Y", auto_pad="NOTSET", dilations=None, group=1, kernel_shape=None, pads=None,
            strides=None),
    _schema("GlobalAveragePool", "X", "Y"),
    _schema("MaxPool", "X", "Y Indices?", auto_pad="NOTSET", ceil_mode=0, dilations=None, kernel_shape=REQUIRED, pads=None,
            storage_order=0, strides=None),
    # reverse of MaxPool: the reference's DefaultMaxPoolBackward reads the forward input and the output gradient
    _schema("MaxPoolGrad", "X dY", "dX", since=1, kernel_shape=REQUIRED, strides=None),
    # Pad in its attribute form: the importer turns the `pads` / `constant_value` inputs of opset 11+ into these when
    # they are known at import time. fusion.fuse_pad_into_conv folds it into the Conv that reads it, as PadConvFusion
    # does (daceml/transformation/pad_conv_fusion.py:13-104); what does not fold runs on the constant-pad kernel (the
    # reference has no expansion for Pad and leaves a stand-alone one to onnxruntime)
    _schema("Pad", "data", "output", since=2, mode="constant", pads=REQUIRED, value=0.0),
    # "mean" / "var" name both inputs and outputs in ONNX; the connectors carry the in_ / out_ prefixes of the
    # reference (tests/test_shared_input_output.py)
    _schema("BatchNormalization", "X scale B in_mean in_var", "Y out_mean? out_var? saved_mean? saved_var?",
            since=9, epsilon=1e-5, momentum=0.9),
    # fused nodes (not in opset 12)
    _schema("LayerNormalization", "X Scale B?", "Y Mean? InvStdDev?", since=17, axis=-1, epsilon=1e-5),
    _schema("SkipLayerNormalization", "input skip gamma beta?", "output mean? inv_std_var? input_skip_bias_sum?",
            since=1, epsilon=1e-5),
    _schema("Gelu", "X", "Y", since=20),
    _schema("BiasGelu", "A B", "C", since=1),
    _schema("Swish", "X", "Y", since=1),
    # a contraction with its neighbours folded in (scale, bias Add, activation, residual Add);
    # produced by the fusion pass, never by an importer
    # InputSum: Inputs__0 summed over the contracted indices (the bias gradient beside a weight gradient)
    _schema("FusedEinsum", "Inputs* Bias? Residual?", "Output PreActivation? InputSum?", since=1, equation=REQUIRED,
            alpha=1.0, activation="none", accumulate=0),
    # Einsum(Q,K) [* scale] -> Softmax(last axis) -> Einsum(P,V) as one node (the scores never reach memory).
    # *_perm: which dimension of that tensor is (batch0, batch1, sequence, head); -1 for an absent batch dim.
    # Mask: added to the scaled scores before the Softmax; broadcasts against [batch.., queries, keys] by the
    # right-aligned rule of Add and must not vary with the query.
    _schema("FusedAttention", "Q K V Mask?", "Output LogSumExp?", since=1, scale=1.0, q_perm=REQUIRED, k_perm=REQUIRED,
            v_perm=REQUIRED, o_perm=REQUIRED),
    _schema("FusedAttentionGrad", "Q K V O LogSumExp dO Mask?", "dQ dK dV", since=1, scale=1.0, q_perm=REQUIRED,
            k_perm=REQUIRED, v_perm=REQUIRED, o_perm=REQUIRED),
    # Conv 1x1 whose input is first multiplied by a per-image, per-channel factor Gate [n, c, 1, 1] (squeeze-excite)
    _schema("GatedConv", "X Gate W B?", "Y", since=1, auto_pad="NOTSET", dilations=None, group=1, kernel_shape=None,
            pads=None, strides=None),
    # pointwise Conv (W_pw [m, c, 1, 1]) + activation followed by a 3x3 depthwise Conv (W_dw [m, 1, 3, 3], padding 1,
    # stride `strides`) + activation: the expanded tensor of an inverted-residual block never reaches memory
    _schema("ExpandDepthwiseConv", "X W_pw B_pw? W_dw B_dw?", "Y", since=1, strides=None, act_pw="none", act_dw="none"),
    # several FusedEinsum nodes of identical equation, shapes, strides and scale, independent of each other, in one
    # launch: Output__i = alpha * einsum(equation, A__i, B__i) [+ Bias__i]
    _schema("GroupedEinsum", "A* B* Bias*?", "Output* InputSum*?", since=1, equation=REQUIRED, alpha=1.0),
    # several independent ReduceSum(all leading axes, keepdims=0) nodes in one launch pair: reduced__i = sum of
    # data__i over every axis but the last (the bias gradients of a backward pass)
    _schema("EinsumSum", "A* B* Residual?", "Output", since=1, equation=REQUIRED, alpha=1.0),
    _schema("MultiReduceSum", "data*", "reduced*", since=1),
    # reduced = ReduceSum(Mul(A, B), axes) with A and B of one shape and `axes` the trailing axes: the product is not
    # written (the gradient of a broadcast factor)
    _schema("MulReduceSum", "A B", "reduced", since=1, axes=REQUIRED, keepdims=1),
    # Y = A * S + T * Scale with S and T holding one value per row of A (A's shape with trailing 1s) and Scale one
    # element: Sum(Mul(A, S), ScaledExpand(T, Scale)) in one pass
    _schema("RowAffine", "A S T Scale?", "Y", since=1),
    # backward nodes emitted by the "hip" BackwardImplementations (names follow the ONNX Runtime
    # training contrib ops)
    _schema("SoftmaxGrad", "dY Y", "dX", since=1, axis=-1),
    # Y = broadcast(X) * Scale to the shape of Y's descriptor (X has Y's rank with extents equal or 1; Scale is one
    # element): the reverse of a mean / sum reduction (ReverseReduce, daceml/autodiff/implementations/dace_nodes.py:13-105)
    # x_shape: the shape X is read with when its descriptor has the size-1 dims squeezed out (keepdims = 0)
    _schema("ScaledExpand", "X Scale", "Y", since=1, x_shape=None),
    # `activation` other than "none": dY is the gradient of activation(BatchNormalization(X)) and B is needed
    _schema("BatchNormalizationGrad", "dY X scale saved_mean saved_var B?", "dX? dscale? dB?", since=1, epsilon=1e-5,
            activation="none"),
    _schema("LayerNormalizationGrad", "Y_grad X scale mean inv_std_var", "X_grad scale_grad bias_grad", since=1,
            axis=-1),
    _schema("GeluGrad", "dY X", "dX", since=1),
    _schema("SwishGrad", "dY X", "dX", since=1),
    _schema("SigmoidGrad", "dY X", "dX", since=1),
    _schema("ReluGrad", "dY X", "dX", since=1),
    _schema("TanhGrad", "dY X", "dX", since=1),
    _schema("ErfGrad", "dY X", "dX", since=1), _schema("SqrtGrad", "dY X", "dX", since=1),
    _schema("ExpGrad", "dY X", "dX", since=1), _schema("LogGrad", "dY X", "dX", since=1),
    _schema("ReciprocalGrad", "dY X", "dX", since=1),
    _schema("ConvGrad", "dY X W", "dX? dW? dB?", since=1, auto_pad="NOTSET", dilations=None, group=1,
            kernel_shape=None, pads=None, strides=None),
]

_default_implementation = {"value": "hip"}


class ONNXOp(Node):
    """Abstract superclass of all ONNX library nodes (daceml/onnx/nodes/onnx_op.py:ONNXOp)."""
    schema: ONNXSchema = None
    implementations: Dict[str, type] = {}
    default_implementation: Optional[str] = None
    default_backward_implementation: Optional[str] = None

    def __init__(self, name: str, *, location=None, **attributes):
        super().__init__(name)
        self.location = location
        self.implementation: Optional[str] = None
        self.backward_implementation: Optional[str] = None
        unknown = set(attributes) - set(self.schema.attributes)
        if unknown:
            raise TypeError("{} has no attribute(s) {}".format(self.schema.name, sorted(unknown)))
        for attr, default in self.schema.attributes.items():
            if attr in attributes:
                setattr(self, attr, attributes[attr])
            elif default is REQUIRED:
                raise ValueError("Expected value for required attribute '{}' of {}".format(attr, self.schema.name))
            else:
                setattr(self, attr, default)
        # required, single connectors are added automatically (onnx_op.py:563-600)
        for p in self.schema.inputs:
            if p.kind == "single":
                self.add_in_connector(p.name)
        for p in self.schema.outputs:
            if p.kind == "single":
                self.add_out_connector(p.name)

    # -- registry ------------------------------------------------------------
    @classmethod
    def register_implementation(cls, name: str, expansion: type):
        cls.implementations[name] = expansion

    # -- edges in ONNX order (onnx_op.py:108-211) ----------------------------
    def _ordered(self, edges, params, conn_of):
        def key(e):
            conn = conn_of(e)
            base, idx = (parse_variadic_param(conn) if "__" in conn else (conn, 0))
            pos = [p.name for p in params].index(base)
            return (pos, idx)
        return sorted(edges, key=key)

    def iter_inputs_in_onnx_order(self, state: SDFGState):
        return self._ordered(state.in_edges(self), self.schema.inputs, lambda e: e.dst_conn)

    def iter_outputs_in_onnx_order(self, state: SDFGState):
        return self._ordered(state.out_edges(self), self.schema.outputs, lambda e: e.src_conn)

    # -- validation ----------------------------------------------------------
    def validate(self, sdfg: SDFG, state: SDFGState):
        """Connector / type checks of onnx_op.py:213-431 that matter on this path."""
        for is_input, params, edges, conns in ((True, self.schema.inputs, state.in_edges(self), self.in_connectors),
                                               (False, self.schema.outputs, state.out_edges(self),
                                                self.out_connectors)):
            names = {p.name: p for p in params}
            seen: Dict[str, List[int]] = {}
            edge_conns = set()
            for e in edges:
                conn = e.dst_conn if is_input else e.src_conn
                if conn is None:
                    raise ValueError("{}: edge without connector".format(self.label))
                edge_conns.add(conn)
                base = conn
                if "__" in conn:
                    base, idx = parse_variadic_param(conn)
                    if base not in names or not names[base].kind.startswith("variadic"):
                        raise ValueError("{}: '{}' is not a variadic parameter of {}".format(
                            self.label, base, self.schema.name))
                    seen.setdefault(base, []).append(idx)
                elif base not in names:
                    raise ValueError("{}: unknown connector '{}' for {}".format(self.label, conn, self.schema.name))
                elif names[base].kind.startswith("variadic"):
                    raise ValueError("{}: variadic parameter '{}' must be numbered".format(self.label, base))
            for p in params:
                if p.kind == "single" and p.name not in edge_conns:
                    raise ValueError("{}: required {} connector '{}' of {} is not connected".format(
                        self.label, "input" if is_input else "output", p.name, self.schema.name))
                if p.kind.startswith("variadic"):
                    idxs = sorted(seen.get(p.name, []))
                    if not idxs and p.kind == "variadic?":
                        continue
                    if not idxs:
                        raise ValueError("{}: variadic parameter '{}' needs at least one edge".format(
                            self.label, p.name))
                    if idxs != list(range(len(idxs))):
                        raise ValueError("{}: variadic parameter '{}' must be numbered 0..n-1 without gaps, got {}"
                                         .format(self.label, p.name, idxs))
            for conn in conns:
                if conn not in edge_conns:
                    raise ValueError("{}: connector '{}' has no edge".format(self.label, conn))
        dtypes = set()
        for e in state.in_edges(self) + state.out_edges(self):
            desc = sdfg.arrays[e.data.data]
            if desc.dtype in (torch.int64, torch.int32, torch.bool):
                continue  # shape / index inputs
            dtypes.add(desc.dtype)
        if self.schema.name != "Cast":
            bad = [d for d in dtypes if d not in FLOAT_DTYPES and d != torch.float64]
            if bad:
                raise TypeError("{}: unsupported element type {}".format(self.label, bad))

    # -- expansion -----------------------------------------------------------
    def selected_implementation(self) -> str:
        return self.implementation or type(self).default_implementation or _default_implementation["value"]

    def expand(self, sdfg: SDFG, state: SDFGState, **kwargs):
        """Expand with the selected implementation (the per-class Expansion wrapper of
        onnx_op.py:668-697). Unlike the reference there is no ONNX Runtime to fall back to: an
        implementation that cannot be applied raises NotApplicable."""
        name = self.selected_implementation()
        impls = type(self).implementations
        if name not in impls:
            raise NotApplicable("{}: no implementation named '{}' for {} (registered: {})".format(
                self.label, name, self.schema.name, sorted(impls)))
        self.validate(sdfg, state)
        impl = impls[name]
        if not impl.forward_can_be_applied(self, state, sdfg):
            raise NotApplicable("{}: implementation '{}' of {} cannot be applied to this node".format(
                self.label, name, self.schema.name))
        return impl.forward(self, state, sdfg, **kwargs)


_ONNX_OPS: Dict[str, type] = {}


def _make_class(schema: ONNXSchema) -> type:
    cls = type("ONNX" + schema.name, (ONNXOp, ), {
        "schema": schema,
        "implementations": {},
        "default_implementation": None,
        "__doc__": "ONNX {} (since opset {}). Inputs: {}. Outputs: {}. Attributes: {}.".format(
            schema.name, schema.since_version, [p.name for p in schema.inputs], [p.name for p in schema.outputs],
            sorted(schema.attributes)),
    })
    return cls


for _s in SCHEMAS:
    _ONNX_OPS[_s.name] = _make_class(_s)
    globals()["ONNX" + _s.name] = _ONNX_OPS[_s.name]


def has_onnx_node(name: str) -> bool:
    """onnx_op.py:716-721."""
    return name in _ONNX_OPS


def get_onnx_node(name: str) -> type:
    """onnx_op.py:724-729."""
    if name not in _ONNX_OPS:
        raise ValueError("Could not find an ONNX node for op '{}'".format(name))
    return _ONNX_OPS[name]


__all__ = ["ONNXOp", "NotApplicable", "parse_variadic_param", "has_onnx_node", "get_onnx_node", "ONNXSchema",
           "ONNXParameter"] + ["ONNX" + s.name for s in SCHEMAS]
