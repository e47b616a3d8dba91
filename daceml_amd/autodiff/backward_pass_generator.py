"""Reverse-mode differentiation of a state made of ONNX library nodes.

The reference's ``BackwardPassGenerator`` (daceml/autodiff/backward_pass_generator.py:526-769) also
differentiates maps and tasklets symbolically; on the library-node path only its registry walk is
involved, and that is what this module provides: select the subgraph between the required inputs and
the given outputs (:616-640), walk it in reverse topological order (:658-769), ask the registry for a
``BackwardImplementation`` per node (:1042-1092), and sum gradient contributions of arrays with
several consumers with an ``ONNXSum`` node (:715-752). Gradient arrays are named ``gradient_<array>``
(:642-648); forward values the reverse nodes read are simply read by name, since forward and backward
live in one SDFG (``add_backward_pass``, daceml/autodiff/autodiff.py:9-58).
"""
from typing import Dict, List, Optional, Sequence, Tuple

import torch

from .. import onnx as donnx
from ..onnx.nodes import ONNXOp
from ..sdfg import SDFG, AccessNode, Array, Node, SDFGState, contiguous_strides
from .base_abc import (AutoDiffException, BackwardContext, BackwardGroup, BackwardResult,
                       find_backward_implementation)


def _root(sdfg: SDFG, name: str) -> str:
    while sdfg.arrays[name].view_of is not None:
        name = sdfg.arrays[name].view_of
    return name


class BackwardPassGenerator:
    def __init__(self, sdfg: SDFG, state: SDFGState, given_gradients: Sequence[str], required_gradients: Sequence[str],
                 backward_sdfg: SDFG, backward_state: SDFGState, grad_dtypes: Optional[Dict[str, torch.dtype]] = None):
        self.sdfg = sdfg
        self.forward_state = state
        self.backward_sdfg = backward_sdfg
        self.backward_state = backward_state
        self.given_gradients = list(given_gradients)
        self.required_gradients = list(required_gradients)
        self.grad_dtypes = dict(grad_dtypes or {})
        self.array_grad_map: Dict[str, str] = {}
        self._contrib: Dict[str, List[str]] = {}      # forward array (root) -> gradient contribution arrays
        self._expected: Dict[str, int] = {}           # forward array (root) -> number of contributions to come
        for name in self.given_gradients + self.required_gradients:
            if name not in sdfg.arrays:
                raise AutoDiffException("array %r is not in the SDFG" % name)
        if backward_sdfg is not sdfg:
            raise AutoDiffException("separate backward SDFGs are not supported: pass backward_sdfg=sdfg")

    # -- names ---------------------------------------------------------------
    def array_grad_name(self, forward_name: str) -> str:
        """``gradient_<name>`` (backward_pass_generator.py:642-648), made unique if that name is taken."""
        if forward_name not in self.array_grad_map:
            name, i = "gradient_" + forward_name, 0
            while name in self.backward_sdfg.arrays:
                i += 1
                name = "gradient_%s_%d" % (forward_name, i)
            self.array_grad_map[forward_name] = name
        return self.array_grad_map[forward_name]

    def grad_dtype(self, forward_name: str) -> torch.dtype:
        return self.grad_dtypes.get(forward_name, self.sdfg.arrays[forward_name].dtype)

    # -- subgraph selection (backward_pass_generator.py:616-640) --------------
    def _subgraph(self) -> List[ONNXOp]:
        st = self.forward_state
        order = [n for n in st.topological_sort() if isinstance(n, ONNXOp)]
        reads = {id(n): {_root(self.sdfg, e.data.data) for e in st.in_edges(n)} for n in order}
        writes = {id(n): {_root(self.sdfg, e.data.data) for e in st.out_edges(n)} for n in order}
        fwd_arrays = {_root(self.sdfg, a) for a in self.required_gradients}
        fwd_nodes = set()
        for n in order:
            if reads[id(n)] & fwd_arrays:
                fwd_nodes.add(id(n))
                fwd_arrays |= writes[id(n)]
        bwd_arrays = {_root(self.sdfg, a) for a in self.given_gradients}
        bwd_nodes = set()
        for n in reversed(order):
            if writes[id(n)] & bwd_arrays:
                bwd_nodes.add(id(n))
                bwd_arrays |= reads[id(n)]
        self._active_arrays = fwd_arrays & bwd_arrays
        return [n for n in order if id(n) in fwd_nodes and id(n) in bwd_nodes]

    # -- main ----------------------------------------------------------------
    def backward(self) -> Dict[str, str]:
        """Generate the backward pass. Returns {forward array: gradient array} for the required gradients."""
        sdfg, st = self.sdfg, self.forward_state
        self._declared = set()
        # the caller passes the gradients of the outputs and receives those of the inputs
        for name in self.given_gradients:
            g = "gradient_" + name
            if g not in sdfg.arrays:
                d = sdfg.arrays[name]
                sdfg.add_array(g, d.shape, self.grad_dtype(name))
            self._declared.add(g)
            self.array_grad_map[name] = g
        for name in self.required_gradients:
            g = "gradient_" + name
            if g not in sdfg.arrays:
                d = sdfg.arrays[name]
                sdfg.add_array(g, d.shape, self.grad_dtype(name))
            self._declared.add(g)
            self.array_grad_map[name] = g

        nodes = self._subgraph()
        if not nodes:
            raise AutoDiffException("no path from the required inputs to the given outputs")
        # how many gradient contributions will each array receive?
        for n in nodes:
            for e in st.in_edges(n):
                r = _root(sdfg, e.data.data)
                if r in self._active_arrays and self._differentiable_input(n, e.dst_conn):
                    self._expected[r] = self._expected.get(r, 0) + 1

        # an output that other nodes of the subgraph also read: the caller's gradient is ONE contribution; the
        # consumers' contributions are summed with it into a transient of its own (never into the caller's
        # buffer), and the producer's reverse node waits for that sum
        ready: Dict[str, str] = {}
        for name in self.given_gradients:
            r = _root(sdfg, name)
            if self._expected.get(r, 0) == 0:
                ready[r] = self.array_grad_map[name]
                continue
            if r != name:
                raise AutoDiffException("output %r is a view of %r, which other nodes read" % (name, r))
            self._expected[r] += 1
            self._contrib[r] = [self.array_grad_map[name]]
            total, i = "gradient_%s_total" % name, 0
            while total in sdfg.arrays:
                i += 1
                total = "gradient_%s_total_%d" % (name, i)
            self.array_grad_map[r] = total
        for n in reversed(nodes):
            self._reverse_node(n, ready)
        result = {}
        for name in self.required_gradients:
            r = _root(sdfg, name)
            if r not in ready:
                raise AutoDiffException("no gradient reached %r" % name)
            result[name] = ready[r]
        return result

    def _differentiable_input(self, node: ONNXOp, conn: str) -> bool:
        non_diff = {"Reshape": {"shape"}}
        return conn not in non_diff.get(node.schema.name, set())

    # -- one node --------------------------------------------------------------
    def _reverse_node(self, node: ONNXOp, ready: Dict[str, str]):
        sdfg, st, bst = self.sdfg, self.forward_state, self.backward_state
        given = []
        for e in st.out_edges(node):
            r = _root(sdfg, e.data.data)
            if r in ready:
                given.append(e.src_conn)
        if not given:
            return  # no gradient flows through this node
        required = [e.dst_conn for e in st.in_edges(node)
                    if _root(sdfg, e.data.data) in self._active_arrays and self._differentiable_input(node, e.dst_conn)]
        impl = find_backward_implementation(sdfg, st, node)
        if impl is None:
            raise AutoDiffException("no applicable BackwardImplementation for %s node %r" % (node.schema.name, node))
        context = BackwardContext(sdfg, st, self.backward_sdfg, bst, self)
        rev, result = impl.backward(node, context, given, required)

        # gradients of the outputs flow in
        for conn in given:
            out_arr = next(iter(st.out_edges_by_connector(node, conn))).data.data
            grad_arr = self._view_like(ready[_root(sdfg, out_arr)], out_arr)
            gconn = result.given_grad_names.get(conn)
            if gconn is None:
                continue
            for tgt, tconn in self._targets(rev, gconn):
                bst.add_edge(bst.add_read(grad_arr), None, tgt, tconn, sdfg.make_array_memlet(grad_arr))
        # gradients of the inputs flow out
        for conn in required:
            in_arr = next(iter(st.in_edges_by_connector(node, conn))).data.data
            root = _root(sdfg, in_arr)
            if conn in result.passthrough:
                out_arr = next(iter(st.out_edges_by_connector(node, result.passthrough[conn]))).data.data
                self._register(root, self._view_like(ready[_root(sdfg, out_arr)], root), ready)
                continue
            gconn = result.required_grad_names.get(conn)
            if gconn is None:
                raise AutoDiffException("%r: the reverse node computes no gradient for input %r" % (node, conn))
            src, sconn = self._source(rev, gconn)
            begin = self._slice_of_root(root, in_arr)
            if begin is not None:
                # the node read a slice of `root`: its gradient is the gradient of the slice with zeros around it -
                # a Pad from a buffer shaped like the slice into a contribution shaped like the root
                fd, rd = sdfg.arrays[in_arr], sdfg.arrays[root]
                part, _ = sdfg.add_transient("%s_slice_%d" % (self.array_grad_name(root), len(self._contrib.get(root, []))),
                                             fd.shape, self.grad_dtype(root))
                bst.add_edge(src, sconn, bst.add_write(part), None, sdfg.make_array_memlet(part))
                target = self._contribution_array(root, root)
                end = [r - b - d for r, b, d in zip(rd.shape, begin, fd.shape)]
                pad = donnx.get_onnx_node("Pad")("scatter_" + part, pads=list(begin) + end, value=0.0, mode="constant")
                bst.add_node(pad)
                pad.add_in_connector("data")
                pad.add_out_connector("output")
                bst.add_edge(bst.add_read(part), None, pad, "data", sdfg.make_array_memlet(part))
                bst.add_edge(pad, "output", bst.add_write(target), None, sdfg.make_array_memlet(target))
                self._register(root, target, ready)
                continue
            target = self._contribution_array(root, in_arr)
            bst.add_edge(src, sconn, bst.add_write(target), None, sdfg.make_array_memlet(target))
            self._register(root, _root(sdfg, target) if sdfg.arrays[target].view_of else target, ready)

    def _targets(self, rev: Node, conn: str) -> List[Tuple[Node, str]]:
        if isinstance(rev, BackwardGroup):
            return rev.inputs.get(conn, [])   # empty when every input gradient is a pass-through of the given one
        return [(rev, conn)]

    def _source(self, rev: Node, conn: str) -> Tuple[Node, str]:
        if isinstance(rev, BackwardGroup):
            return rev.outputs[conn]
        return rev, conn

    def _slice_of_root(self, root: str, array: str) -> Optional[List[int]]:
        """Where `array` starts along each axis of `root` when it is a rectangular part of it (a view with the root's
        own strides that covers fewer elements); None when it is the root or a view of all of it."""
        fd, rd = self.sdfg.arrays[array], self.sdfg.arrays[root]
        if array == root or fd.view_of is None or fd.total_size == rd.total_size:
            return None
        if len(fd.shape) != len(rd.shape) or tuple(fd.strides) != tuple(rd.strides) or not rd.is_contiguous():
            raise AutoDiffException("%r is a part of %r that is not a rectangular slice with unit steps: no gradient"
                                    % (array, root))
        begin, rest = [], fd.view_offset
        for stride in rd.strides:
            begin.append(rest // stride if stride else 0)
            rest -= begin[-1] * stride if stride else 0
        if rest or any(b + d > r for b, d, r in zip(begin, fd.shape, rd.shape)):
            raise AutoDiffException("%r does not lie inside %r as a rectangle" % (array, root))
        return begin

    # -- gradient buffers --------------------------------------------------------
    def _view_like(self, grad_array: str, forward_array: str) -> str:
        """The gradient buffer `grad_array`, seen with the shape of `forward_array` (a dense reshape)."""
        gd, fd = self.sdfg.arrays[grad_array], self.sdfg.arrays[forward_array]
        if gd.shape == fd.shape:
            return grad_array
        if gd.total_size != fd.total_size or not fd.is_contiguous():
            raise AutoDiffException("cannot view gradient %r with the layout of %r" % (grad_array, forward_array))
        name, _ = self.sdfg.add_view("%s_as_%s" % (grad_array, forward_array), grad_array, fd.shape,
                                     contiguous_strides(fd.shape))
        return name

    def _contribution_array(self, root: str, read_as: str) -> str:
        """Where a reverse node writes its gradient for `root`, shaped like the array it read."""
        sdfg = self.sdfg
        if self._expected.get(root, 1) <= 1:
            base = self.array_grad_name(root)
            if base not in sdfg.arrays:
                sdfg.add_array(base, sdfg.arrays[root].shape, self.grad_dtype(root), transient=True)
        else:
            idx = len(self._contrib.get(root, []))
            base, _ = sdfg.add_transient("%s_contribution_%d" % (self.array_grad_name(root), idx),
                                         sdfg.arrays[root].shape, self.grad_dtype(root))
        return self._view_like(base, read_as)

    def _register(self, root: str, grad_buffer: str, ready: Dict[str, str]):
        """Record a contribution; once all have arrived, publish the gradient of `root`."""
        sdfg, bst = self.sdfg, self.backward_state
        lst = self._contrib.setdefault(root, [])
        lst.append(grad_buffer)
        if len(lst) < self._expected.get(root, 1):
            return
        if len(lst) == 1:
            final = self.array_grad_name(root)
            if lst[0] != final:
                if final in self._declared:
                    # a passthrough reached a caller-visible gradient: it has to be materialised
                    ident = donnx.ONNXIdentity("copy_" + final)
                    bst.add_node(ident)
                    bst.add_edge(bst.add_read(lst[0]), None, ident, "input", sdfg.make_array_memlet(lst[0]))
                    bst.add_edge(ident, "output", bst.add_write(final), None, sdfg.make_array_memlet(final))
                else:
                    self.array_grad_map[root] = lst[0]
                    final = lst[0]
            ready[root] = final
            return
        final = self.array_grad_name(root)
        if final not in sdfg.arrays:
            sdfg.add_array(final, sdfg.arrays[root].shape, self.grad_dtype(root), transient=True)
        dt = sdfg.arrays[final].dtype
        if any(sdfg.arrays[c].dtype != dt for c in lst):
            raise AutoDiffException("gradient contributions of %r have different dtypes" % root)
        # ONNXSum over the contributions (backward_pass_generator.py:715-752)
        summ = donnx.ONNXSum("accumulate_" + final)
        bst.add_node(summ)
        for i, c in enumerate(lst):
            summ.add_in_connector("data_0__%d" % i)
            bst.add_edge(bst.add_read(c), None, summ, "data_0__%d" % i, sdfg.make_array_memlet(c))
        bst.add_edge(summ, "sum", bst.add_write(final), None, sdfg.make_array_memlet(final))
        ready[root] = final


def add_backward_pass(sdfg: SDFG, state: SDFGState, outputs: Sequence[str], inputs: Sequence[str],
                      grad_dtypes: Optional[Dict[str, torch.dtype]] = None) -> Dict[str, str]:
    """Add a state with the backward pass after `state` (daceml/autodiff/autodiff.py:9-58).

    The caller then passes ``gradient_<output>`` for every output and receives ``gradient_<input>`` for
    every input. ``grad_dtypes`` overrides the gradient element type per forward array (fp32 master
    gradients for fp16 parameters)."""
    backward_state = sdfg.add_state(state.label + "_backward")
    gen = BackwardPassGenerator(sdfg, state, outputs, inputs, sdfg, backward_state, grad_dtypes)
    return gen.backward()
