"""Import of an ONNX model into an SDFG of ONNX library nodes.

Follows daceml/onnx/onnx_importer.py:107-338: one state holding one library node per graph node, access nodes
named by ``clean_onnx_name``, ``Constant`` nodes turned into constant arrays at import, variadic connectors
numbered ``<name>__<i>``, model outputs renamed ``__return`` / ``__return_<i>``. Where the reference calls
``onnx.shape_inference`` and ``onnxsim`` (constant folding of the Shape / Gather / Unsqueeze / Concat chains the
exporter emits around ``view``), this importer carries static shapes itself: every tensor gets its shape from a
per-operator rule, and nodes whose inputs are all known at import time (constants and shape arithmetic, never
parameters) are evaluated with NumPy instead of becoming library nodes.
"""
import re
from typing import Dict, List, Optional, Sequence, Tuple, Union

import numpy as np
import torch

from . import nodes as donnx
from . import proto
from ..sdfg import SDFG, SDFGState

_NP_TO_TORCH = {np.dtype(np.float16): torch.float16, np.dtype(np.float32): torch.float32,
                np.dtype(np.float64): torch.float64, np.dtype(np.int64): torch.int64,
                np.dtype(np.int32): torch.int32, np.dtype(np.bool_): torch.bool}
_ONNX_TO_TORCH = {1: torch.float32, 10: torch.float16, 11: torch.float64, 7: torch.int64, 6: torch.int32,
                  9: torch.bool}
_TORCH_TO_NP = {v: k for k, v in _NP_TO_TORCH.items()}


def clean_onnx_name(name: str) -> str:
    """A valid array / node name from an ONNX name (daceml/onnx/converters.py:204-211)."""
    if re.match("^[0-9]", name):
        name = "ONNX_" + name
    return name.replace(".", "DOT").replace(":", "COLON").replace("/", "SLASH").replace("-", "DASH")


class UnsupportedModel(ValueError):
    pass


def _broadcast(a: Sequence[int], b: Sequence[int]) -> Tuple[int, ...]:
    out = []
    for i in range(1, max(len(a), len(b)) + 1):
        x = a[-i] if i <= len(a) else 1
        y = b[-i] if i <= len(b) else 1
        if x != y and x != 1 and y != 1:
            raise UnsupportedModel("shapes %s and %s do not broadcast" % (tuple(a), tuple(b)))
        out.append(max(x, y))
    return tuple(reversed(out))


def _axes(axes, rank: int) -> List[int]:
    if axes is None:
        return list(range(rank))
    return sorted(a % rank for a in axes)


# evaluated at import time when every input is known (shape arithmetic and constants)
_FOLDABLE = {
    "Add": np.add, "Sub": np.subtract, "Mul": np.multiply, "Neg": np.negative, "Sqrt": np.sqrt,
    "Equal": np.equal, "Identity": lambda x: x,
}


class ONNXModel:
    """Loads an ONNX model (bytes, path, file object or a decoded ``proto.ModelProto``) into ``self.sdfg``.

    ``inputs`` / ``outputs``: names the caller passes / receives (outputs already renamed to ``__return*``);
    ``weights``: initializer name -> tensor, passed automatically by ``__call__``. Arrays are named
    ``clean_onnx_name(onnx name)``. ``parameters_as_inputs``: initializer names that stay out of ``weights``
    because the caller passes live tensors for them (what DaceModule does with module parameters,
    daceml/torch/module.py:289-312)."""
    def __init__(self, name: str, model, cuda: bool = True, auto_optimize: bool = True,
                 parameters_as_inputs: Optional[Sequence[str]] = None, training: bool = False):
        if not isinstance(model, proto.ModelProto):
            model = proto.load_model(model)
        self.model = model
        self.cuda = cuda
        self.do_auto_optimize = auto_optimize
        self.training = training
        self.opset = model.opset_import.get("", 12)
        graph = model.graph
        self.sdfg = SDFG(name)
        self.state: SDFGState = self.sdfg.add_state("main")
        self.sdfg._parent_onnx_model = self
        self.weights: Dict[str, torch.Tensor] = {}
        self.inputs: List[str] = []
        self.outputs: List[str] = []
        self._known: Dict[str, np.ndarray] = {}     # values available at import time, by ONNX name
        self._alias: Dict[str, str] = {}            # ONNX name -> ONNX name it is identical to
        self._access = {}
        self._compiled = None
        external = set(parameters_as_inputs or ())

        init_names = {t.name for t in graph.initializer}
        for value in graph.input:
            if value.name in init_names:
                continue                 # keep_initializers_as_inputs: described by the initializer itself
            if value.shape is None or any(not isinstance(d, int) for d in value.shape):
                raise UnsupportedModel("input %r needs a static shape, got %s" % (value.name, value.shape))
            if value.elem_type not in _ONNX_TO_TORCH:
                raise UnsupportedModel("input %r has unsupported element type %d" % (value.name, value.elem_type))
            self.inputs.append(value.name)
            self.sdfg.add_array(clean_onnx_name(value.name), tuple(value.shape), _ONNX_TO_TORCH[value.elem_type])
        for t in graph.initializer:
            arr = t.array
            if arr.dtype not in _NP_TO_TORCH:
                raise UnsupportedModel("initializer %r has unsupported dtype %s" % (t.name, arr.dtype))
            self.sdfg.add_array(clean_onnx_name(t.name), tuple(arr.shape), _NP_TO_TORCH[arr.dtype])
            if t.name in external:
                self.inputs.append(t.name)
            else:
                self.weights[t.name] = torch.from_numpy(np.array(arr))
            if arr.dtype.kind in "iub":
                self._known[t.name] = arr     # integer initializers are shape data, never trained
        self.sdfg.arg_names = [clean_onnx_name(i) for i in self.inputs]

        for i, node in enumerate(graph.node):
            self._import_node(i, node)

        for i, out in enumerate(graph.output):
            src = self._resolve(out.name)
            clean = clean_onnx_name(src)
            if clean not in self.sdfg.arrays or not self.sdfg.arrays[clean].transient:
                raise UnsupportedModel("output %r is not produced by a node of the graph" % out.name)
            new = "__return" if len(graph.output) == 1 else "__return_%d" % i
            desc = self.sdfg.arrays[clean]
            if desc.view_of is not None:
                # an output that is a part of another array (a Slice): the caller's buffer gets a copy of it
                self.sdfg.add_array(new, tuple(desc.shape), desc.dtype, transient=True)
                copy = donnx.get_onnx_node("Identity")("copy_%s" % new)
                self.state.add_node(copy)
                copy.add_in_connector("input")
                copy.add_out_connector("output")
                self.state.add_edge(self._access_node(clean, False), None, copy, "input", self.sdfg.make_array_memlet(clean))
                self.state.add_edge(copy, "output", self._access_node(new, True), None, self.sdfg.make_array_memlet(new))
            else:
                self._rename_array(clean, new)
            self.sdfg.arrays[new].transient = False
            self.outputs.append(new)
        self._drop_unreferenced()

    # ------------------------------------------------------------------ graph construction
    def _drop_unreferenced(self):
        """Initializers that only fed import-time evaluation (shape data) have no access node: they are not
        arguments of the program. Graph inputs stay, used or not, because the caller passes them."""
        used = {e.data.data for e in self.state.edges()}
        keep = {clean_onnx_name(n) for n in self.inputs} | set(self.outputs)
        for name in [n for n in self.sdfg.arrays if n not in used and n not in keep]:
            del self.sdfg.arrays[name]
            self.sdfg.constants.pop(name, None)
            self.sdfg.constants_exact.pop(name, None)
        self.weights = {k: v for k, v in self.weights.items() if clean_onnx_name(k) in self.sdfg.arrays}

    def _resolve(self, name: str) -> str:
        while name in self._alias:
            name = self._alias[name]
        return name

    def _rename_array(self, old: str, new: str):
        desc = self.sdfg.arrays.pop(old)
        self.sdfg.arrays[new] = desc
        for e in self.state.edges():
            if e.data.data == old:
                e.data.data = new
        for n in self.state.nodes():
            if getattr(n, "data", None) == old:
                n.data = new
                n.label = new

    def _desc(self, name: str):
        """Descriptor of an ONNX value, materialising import-time values as constant arrays."""
        name = self._resolve(name)
        clean = clean_onnx_name(name)
        if clean not in self.sdfg.arrays:
            if name not in self._known:
                raise UnsupportedModel("value %r is used before it is produced" % name)
            self._materialise(name)
        return self.sdfg.arrays[clean]

    def _materialise(self, name: str):
        arr = np.asarray(self._known[name])
        if arr.dtype not in _NP_TO_TORCH:
            raise UnsupportedModel("constant %r has unsupported dtype %s" % (name, arr.dtype))
        clean = clean_onnx_name(name)
        t = torch.from_numpy(np.array(arr))
        self.sdfg.add_array(clean, tuple(arr.shape), t.dtype)
        self.sdfg.add_constant(clean, t)
        if arr.size == 1:
            self.sdfg.constants_exact[clean] = float(arr.reshape(-1)[0])

    def _shape_of(self, name: str) -> Tuple[int, ...]:
        name = self._resolve(name)
        if name in self._known and clean_onnx_name(name) not in self.sdfg.arrays:
            return tuple(np.asarray(self._known[name]).shape)
        return tuple(self._desc(name).shape)

    def _dtype_of(self, name: str) -> torch.dtype:
        name = self._resolve(name)
        if name in self._known and clean_onnx_name(name) not in self.sdfg.arrays:
            return _NP_TO_TORCH[np.asarray(self._known[name]).dtype]
        return self._desc(name).dtype

    def _access_node(self, clean: str, write: bool):
        if clean not in self._access:
            self._access[clean] = self.state.add_write(clean) if write else self.state.add_read(clean)
        return self._access[clean]

    def _import_node(self, idx: int, node: proto.NodeProto):
        op = node.op_type
        attrs = {a.name: a.value for a in node.attribute}
        ins = [self._resolve(n) if n else "" for n in node.input]

        if op == "Constant":
            # importer rule of the reference (onnx_importer.py:205-233): exactly one value attribute, no inputs
            if len(attrs) != 1 or ins or len(node.output) != 1:
                raise UnsupportedModel("Constant node %r must have one attribute, no inputs and one output" % node.name)
            key, value = next(iter(attrs.items()))
            if key not in ("value", "value_float", "value_floats", "value_int", "value_ints"):
                raise UnsupportedModel("Constant node %r: attribute %r is not supported" % (node.name, key))
            dt = {"value_float": np.float32, "value_floats": np.float32, "value_int": np.int64,
                  "value_ints": np.int64}.get(key)
            self._known[node.output[0]] = np.asarray(value) if dt is None else np.asarray(value, dtype=dt)
            return
        if self._fold(op, node, ins, attrs):
            return
        if op == "Slice":
            self._import_slice(node, ins, attrs)
            return
        if op in ("Dropout", ) and (not self.training or float(attrs.get("ratio", 0.5)) == 0.0):
            self._alias[node.output[0]] = ins[0]     # identity outside training; a mask output is never read
            return
        if op == "Flatten":
            axis = int(attrs.get("axis", 1))
            shp = self._shape_of(ins[0])
            axis = axis % (len(shp) + 1) if axis < 0 else axis
            op, attrs = "Reshape", {}
            ins = ins[:1]
            out_shapes = [(int(np.prod(shp[:axis], dtype=np.int64)), int(np.prod(shp[axis:], dtype=np.int64)))]
            out_dtypes = [self._dtype_of(ins[0])]
        else:
            if not donnx.has_onnx_node(op) or node.domain not in ("", "ai.onnx"):
                raise UnsupportedModel("Unsupported ONNX operator: '%s'" % op)
            out_shapes, out_dtypes, ins, attrs = self._infer(op, node, ins, attrs)

        if op == "BatchNormalization":
            attrs = {k: v for k, v in attrs.items() if k in ("epsilon", "momentum")}   # drops opset-7 `spatial`
        label = clean_onnx_name(node.name) if node.name else "%s_%d" % (op, idx)
        cls = donnx.get_onnx_node(op)
        op_node = cls(label, **attrs)
        self.state.add_node(op_node)
        for kind, names in (("in", ins), ("out", list(node.output))):
            params = op_node.schema.inputs if kind == "in" else op_node.schema.outputs
            for i, name in enumerate(names):
                if not name:
                    continue           # an omitted optional input
                # connector naming of the reference importer (onnx_importer.py:259-281)
                if i >= len(params):
                    if not params or not params[-1].kind.startswith("variadic"):
                        raise UnsupportedModel("%s node %r has more %sputs than its schema" % (op, node.name, kind))
                    conn = "%s__%d" % (params[-1].name, i - len(params) + 1)
                elif params[i].kind.startswith("variadic"):
                    conn = params[i].name + "__0"
                else:
                    conn = params[i].name
                if kind == "in":
                    self._desc(name)
                    clean = clean_onnx_name(name)
                    if conn not in op_node.in_connectors:
                        op_node.add_in_connector(conn)
                    self.state.add_edge(self._access_node(clean, False), None, op_node, conn,
                                        self.sdfg.make_array_memlet(clean))
                else:
                    if i >= len(out_shapes):
                        continue       # an optional output the shape rule does not produce (never read)
                    clean = clean_onnx_name(name)
                    self.sdfg.add_array(clean, tuple(int(d) for d in out_shapes[i]), out_dtypes[i], transient=True)
                    if conn not in op_node.out_connectors:
                        op_node.add_out_connector(conn)
                    self.state.add_edge(op_node, conn, self._access_node(clean, True), None,
                                        self.sdfg.make_array_memlet(clean))

    def _import_slice(self, node, ins: List[str], attrs):
        """A Slice of run-time data whose bounds are known now (the exporter slices the packed q / k / v projection
        weight of ``nn.MultiheadAttention`` this way) becomes a view of its input: same buffer, an offset, strides
        multiplied by the steps. No node, no copy; whether a reader can take the strides is that reader's business."""
        known = lambda i: len(ins) > i and ins[i] and ins[i] in self._known  # noqa: E731
        if "starts" in attrs:                                  # opset < 10: attributes
            starts, ends = list(attrs["starts"]), list(attrs["ends"])
            axes = list(attrs["axes"]) if "axes" in attrs else list(range(len(starts)))
            steps = [1] * len(starts)
        else:
            if not (known(1) and known(2)) or (len(ins) > 3 and ins[3] and not known(3)) or \
                    (len(ins) > 4 and ins[4] and not known(4)):
                raise UnsupportedModel("Slice node %r: the bounds must be known at import time" % node.name)
            starts = np.asarray(self._known[ins[1]]).reshape(-1).tolist()
            ends = np.asarray(self._known[ins[2]]).reshape(-1).tolist()
            axes = np.asarray(self._known[ins[3]]).reshape(-1).tolist() if known(3) else list(range(len(starts)))
            steps = np.asarray(self._known[ins[4]]).reshape(-1).tolist() if known(4) else [1] * len(starts)
        d = self._desc(ins[0])
        shape, strides, offset = list(d.shape), list(d.strides), 0
        for start, end, axis, step in zip(starts, ends, axes, steps):
            axis = int(axis) % len(shape)
            if int(step) <= 0:
                raise UnsupportedModel("Slice node %r: step %d is not supported" % (node.name, step))
            # clamping rule of the ONNX specification for positive steps
            n = shape[axis]
            lo, hi = int(start), int(end)
            lo = min(max(lo + n if lo < 0 else lo, 0), n)
            hi = min(max(hi + n if hi < 0 else hi, 0), n)
            offset += lo * strides[axis]
            shape[axis] = max(0, -(-(hi - lo) // int(step)))
            strides[axis] *= int(step)
        self.sdfg.add_view(clean_onnx_name(node.output[0]), clean_onnx_name(self._resolve(ins[0])), tuple(shape),
                           tuple(strides), offset, find_new_name=False)

    # ------------------------------------------------------------------ import-time evaluation
    def _fold(self, op: str, node, ins: List[str], attrs) -> bool:
        """Evaluates shape arithmetic and constant expressions; returns True when the node was consumed."""
        out = node.output[0]
        if op == "Shape":
            self._known[out] = np.asarray(self._shape_of(ins[0]), dtype=np.int64)
            return True
        if any(n and n not in self._known for n in ins) or not ins:
            return False
        if any(clean_onnx_name(n) in self.sdfg.arrays and self._known[n].dtype.kind == "f" for n in ins if n):
            return False       # floating-point data that already lives in the graph stays there
        v = [np.asarray(self._known[n]) if n else None for n in ins]
        if op in _FOLDABLE:
            r = _FOLDABLE[op](*v)
        elif op == "Div":
            r = v[0] // v[1] if v[0].dtype.kind in "iu" else v[0] / v[1]
        elif op == "Gather":
            r = np.take(v[0], v[1], axis=int(attrs.get("axis", 0)))
        elif op == "Unsqueeze":
            r = v[0]
            for a in sorted(attrs["axes"] if "axes" in attrs else v[1].tolist()):
                r = np.expand_dims(r, a)
        elif op == "Squeeze":
            axes = attrs.get("axes") if "axes" in attrs else (v[1].tolist() if len(v) > 1 else None)
            r = np.squeeze(v[0], axis=None if axes is None else tuple(axes))
        elif op == "Concat":
            r = np.concatenate([np.atleast_1d(x) for x in v], axis=int(attrs["axis"]))
        elif op == "Cast":
            to = int(attrs["to"])
            if to not in proto.TENSOR_DTYPES:
                return False
            r = v[0].astype(proto.TENSOR_DTYPES[to])
        elif op == "Slice":
            if len(v) < 3:
                return False
            starts, ends = v[1].tolist(), v[2].tolist()
            axes = v[3].tolist() if len(v) > 3 and v[3] is not None else list(range(len(starts)))
            steps = v[4].tolist() if len(v) > 4 and v[4] is not None else [1] * len(starts)
            idx = [slice(None)] * v[0].ndim
            for s, e, a, st in zip(starts, ends, axes, steps):
                idx[a] = slice(s, e, st)
            r = v[0][tuple(idx)]
        elif op == "Reshape":
            r = v[0].reshape([int(d) for d in v[1].tolist()])
        elif op == "Transpose":
            r = np.transpose(v[0], attrs.get("perm"))
        elif op == "ConstantOfShape":
            fill = attrs.get("value")
            fill = np.zeros((), np.float32) if fill is None else np.asarray(fill).reshape(())
            r = np.full(tuple(v[0].tolist()), fill, dtype=fill.dtype)
        else:
            return False
        self._known[out] = np.asarray(r)
        return True

    # ------------------------------------------------------------------ shapes
    def _infer(self, op: str, node, ins: List[str], attrs):
        """Output shapes and dtypes of a library node; may drop inputs that were consumed at import time."""
        shp = [self._shape_of(n) if n else None for n in ins]
        dt = self._dtype_of(ins[0])
        attrs = dict(attrs)
        if op in ("Add", "Sub", "Mul", "Div", "Pow"):
            return [_broadcast(shp[0], shp[1])], [dt], ins, attrs
        if op in ("Sqrt", "Relu", "Sigmoid", "Reciprocal", "Erf", "Exp", "Log", "Tanh", "Identity", "Softmax",
                  "LogSoftmax", "Gelu", "Swish"):
            return [shp[0]], [dt], ins, attrs
        if op == "Sum":
            if any(s != shp[0] for s in shp):
                raise UnsupportedModel("Sum node %r: operands of different shapes %s" % (node.name, shp))
            return [shp[0]], [dt], ins, attrs
        if op == "Cast":
            to = int(attrs["to"])
            if to not in _ONNX_TO_TORCH:
                raise UnsupportedModel("Cast node %r: unsupported target type %d" % (node.name, to))
            return [shp[0]], [_ONNX_TO_TORCH[to]], ins, attrs
        if op == "MatMul":
            a, b = shp
            if len(a) < 2 or len(b) < 2:
                raise UnsupportedModel("MatMul node %r: 1-D operands are not supported" % node.name)
            if a[-1] != b[-2]:
                raise UnsupportedModel("MatMul node %r: %s x %s" % (node.name, a, b))
            return [_broadcast(a[:-2], b[:-2]) + (a[-2], b[-1])], [dt], ins, attrs
        if op == "Gemm":
            a, b = shp[0], shp[1]
            if len(a) != 2 or len(b) != 2:
                raise UnsupportedModel("Gemm node %r needs 2-D operands" % node.name)
            m, k = (a[1], a[0]) if attrs.get("transA", 0) else a
            k2, n = (b[1], b[0]) if attrs.get("transB", 0) else b
            if k != k2:
                raise UnsupportedModel("Gemm node %r: inner extents %d and %d" % (node.name, k, k2))
            return [(m, n)], [dt], ins, attrs
        if op in ("ReduceMean", "ReduceSum", "ReduceMax", "ReduceMin"):
            axes = attrs.get("axes")
            if axes is None and len(ins) > 1 and ins[1]:        # opset 13+: axes as an input
                axes = np.asarray(self._known[ins[1]]).tolist()
                attrs["axes"] = axes
                ins = ins[:1]
            ax = _axes(axes, len(shp[0]))
            keep = int(attrs.get("keepdims", 1))
            out = [1 if i in ax else d for i, d in enumerate(shp[0])] if keep else \
                [d for i, d in enumerate(shp[0]) if i not in ax]
            return [tuple(out)], [dt], ins, attrs
        if op == "Transpose":
            perm = attrs.get("perm") or list(reversed(range(len(shp[0]))))
            attrs["perm"] = list(perm)
            return [tuple(shp[0][p] for p in perm)], [dt], ins, attrs
        if op == "Reshape":
            if len(ins) < 2 or ins[1] not in self._known:
                raise UnsupportedModel("Reshape node %r: the target shape must be known at import time" % node.name)
            target = [int(d) for d in np.asarray(self._known[ins[1]]).tolist()]
            target = [shp[0][i] if d == 0 else d for i, d in enumerate(target)]
            total = int(np.prod(shp[0], dtype=np.int64))
            if -1 in target:
                rest = int(np.prod([d for d in target if d != -1], dtype=np.int64))
                target[target.index(-1)] = total // max(rest, 1)
            if int(np.prod(target, dtype=np.int64)) != total:
                raise UnsupportedModel("Reshape node %r: %s -> %s" % (node.name, shp[0], target))
            return [tuple(target)], [dt], ins[:1], attrs
        if op == "Conv":
            x, w = shp[0], shp[1]
            nsp = len(x) - 2
            if attrs.get("auto_pad", "NOTSET") != "NOTSET":
                raise UnsupportedModel("Conv node %r: auto_pad %r is not supported" % (node.name, attrs["auto_pad"]))
            strides = attrs.get("strides") or [1] * nsp
            dil = attrs.get("dilations") or [1] * nsp
            pads = attrs.get("pads") or [0] * (2 * nsp)
            # output extent rule of daceml/onnx/shape_inference/symbolic_shape_infer.py:466-526
            out = [(x[2 + i] + pads[i] + pads[nsp + i] - ((w[2 + i] - 1) * dil[i] + 1)) // strides[i] + 1
                   for i in range(nsp)]
            return [(x[0], w[0]) + tuple(out)], [dt], ins, attrs
        if op == "GlobalAveragePool":
            return [tuple(shp[0][:2]) + (1, ) * (len(shp[0]) - 2)], [dt], ins, attrs
        if op == "MaxPool":
            x = shp[0]
            nsp = len(x) - 2
            k = list(attrs["kernel_shape"])
            strides = list(attrs.get("strides") or [1] * nsp)
            pads = list(attrs.get("pads") or [0] * (2 * nsp))
            dil = list(attrs.get("dilations") or [1] * nsp)
            if attrs.get("auto_pad", "NOTSET") != "NOTSET":
                raise UnsupportedModel("MaxPool node %r: auto_pad %r is not supported" % (node.name, attrs["auto_pad"]))
            out = []
            for i in range(nsp):
                span = x[2 + i] + pads[i] + pads[nsp + i] - ((k[i] - 1) * dil[i] + 1)
                out.append((-(-span // strides[i]) if int(attrs.get("ceil_mode", 0)) else span // strides[i]) + 1)
            return [tuple(x[:2]) + tuple(out)], [dt], ins, attrs
        if op == "Pad":
            # opset 11+: pads and the fill value are inputs; they become attributes, and have to be known now
            mode = attrs.get("mode", "constant")
            mode = mode.decode() if isinstance(mode, bytes) else str(mode)
            pads = attrs.get("pads")
            if pads is None:
                if len(ins) < 2 or ins[1] not in self._known:
                    raise UnsupportedModel("Pad node %r: the pads must be known at import time" % node.name)
                pads = np.asarray(self._known[ins[1]]).reshape(-1).tolist()
            value = float(attrs.get("value", 0.0))
            if len(ins) > 2 and ins[2]:
                if ins[2] not in self._known:
                    raise UnsupportedModel("Pad node %r: the fill value must be known at import time" % node.name)
                value = float(np.asarray(self._known[ins[2]]).reshape(-1)[0])
            pads = [int(p) for p in pads]
            rank = len(shp[0])
            if len(pads) != 2 * rank or any(p < 0 for p in pads):
                raise UnsupportedModel("Pad node %r: pads %s on a tensor of rank %d" % (node.name, pads, rank))
            out = tuple(d + pads[i] + pads[rank + i] for i, d in enumerate(shp[0]))
            return [out], [dt], ins[:1], {"mode": mode, "pads": pads, "value": value}
        if op == "LayerNormalization":
            return [shp[0]], [dt], ins, attrs
        if op == "BatchNormalization":
            # Y, then out_mean, out_var, saved_mean, saved_var when the node is in its training form
            n_out = 5 if len([o for o in node.output if o]) > 1 else 1
            return [shp[0]] + [(shp[0][1], )] * (n_out - 1), [dt] * n_out, ins, attrs
        raise UnsupportedModel("no shape rule for ONNX operator '%s' (node %r)" % (op, node.name))

    # ------------------------------------------------------------------ execution
    def auto_optimize(self):
        from ..transformation import fusion
        return fusion.auto_optimize(self.sdfg, training=self.training)

    def compile_and_init(self, device=None):
        """Expands the library nodes and binds the kernels (daceml/onnx/onnx_importer.py:452-480)."""
        from ..runtime import CompiledSDFG
        if self._compiled is None:
            if self.do_auto_optimize:
                self.auto_optimize()
            self._compiled = CompiledSDFG(self.sdfg, device=device)
            dev = self._compiled.device
            self._device_weights = {clean_onnx_name(k): v.to(dev) for k, v in self.weights.items()
                                    if clean_onnx_name(k) in self._compiled.arglist()}
        return self._compiled

    def __call__(self, *args, **kwargs) -> Union[torch.Tensor, Tuple[torch.Tensor, ...]]:
        """Runs the model on tensors given positionally (in ``inputs`` order) or by ONNX name; returns the output
        tensor, or a tuple of them (daceml/onnx/onnx_importer.py:482-560)."""
        prog = self.compile_and_init()
        given = dict(zip(self.inputs, args))
        if len(args) > len(self.inputs):
            raise TypeError("expected at most %d positional inputs, got %d" % (len(self.inputs), len(args)))
        dup = set(given) & set(kwargs)
        if dup:
            raise TypeError("inputs given twice: %s" % sorted(dup))
        given.update(kwargs)
        missing = [n for n in self.inputs if n not in given]
        if missing or set(given) - set(self.inputs):
            raise TypeError("missing inputs %s, unknown inputs %s" % (missing, sorted(set(given) - set(self.inputs))))
        call = dict(self._device_weights)
        needed = prog.arglist()
        for n, t in given.items():
            clean = clean_onnx_name(n)
            if clean in needed:
                call[clean] = t.contiguous()
        outs = []
        for o in self.outputs:
            d = self.sdfg.arrays[o]
            t = torch.empty(d.shape, dtype=d.dtype, device=prog.device)
            call[o] = t
            outs.append(t)
        prog(**call)
        return outs[0] if len(outs) == 1 else tuple(outs)
