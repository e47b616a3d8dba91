"""A deliberately small stand-in for the part of DaCe's SDFG API that DaCeML's ONNX library-node
path touches: data descriptors, one-state graphs of access nodes and library nodes, and memlet
edges between connectors.

The reference builds on `dace.SDFG` / `dace.SDFGState` (third-party, not available here). The
method names below follow DaCe's (``add_array``, ``add_transient``, ``add_state``, ``add_read``,
``add_write``, ``add_edge``, ``in_edges``, ``out_edges``, ``make_array_memlet`` ...) so that the
implementations in ``daceml_amd.onnx.op_implementations`` read like the reference's
(daceml/onnx/op_implementations/*.py) and port to real DaCe with a search-and-replace of imports.
"""
import copy
import dataclasses
from typing import Dict, Iterable, List, Optional, Sequence, Tuple

import torch

FLOAT_DTYPES = (torch.float16, torch.float32)


def contiguous_strides(shape: Sequence[int]) -> Tuple[int, ...]:
    strides, s = [], 1
    for ext in reversed(tuple(shape)):
        strides.append(s)
        s *= int(ext)
    return tuple(reversed(strides))


class Array:
    """Data descriptor (dace.data.Array): shape, dtype, element strides, transient flag.

    ``view_of`` / ``view_offset`` mark a descriptor that aliases (part of) another array's buffer;
    that is how a folded Transpose / Reshape is represented without a copy.
    """
    def __init__(self, shape, dtype, transient=False, strides=None, view_of: Optional[str] = None,
                 view_offset: int = 0):
        self.shape = tuple(int(s) for s in shape)
        self.dtype = dtype
        self.transient = transient
        self.strides = tuple(int(s) for s in strides) if strides is not None else contiguous_strides(self.shape)
        self.view_of = view_of
        self.view_offset = int(view_offset)
        #: a transient that holds data across calls (AllocationLifetime.Persistent in DaCe): a parameter snapshot
        self.persistent = False

    @property
    def total_size(self) -> int:
        n = 1
        for s in self.shape:
            n *= s
        return n

    def is_contiguous(self) -> bool:
        return self.strides == contiguous_strides(self.shape) or self.total_size <= 1

    def __repr__(self):
        return "Array(%s, %s%s%s)" % (self.shape, str(self.dtype).replace("torch.", ""),
                                      ", transient" if self.transient else "",
                                      ", view_of=%s" % self.view_of if self.view_of else "")


@dataclasses.dataclass
class Memlet:
    data: str


class Node:
    """Base of everything that lives in a state."""
    def __init__(self, label: str):
        self.label = label
        self.in_connectors: Dict[str, None] = {}
        self.out_connectors: Dict[str, None] = {}

    def add_in_connector(self, name: str):
        self.in_connectors[name] = None
        return True

    def add_out_connector(self, name: str):
        self.out_connectors[name] = None
        return True

    def __repr__(self):
        return "%s(%s)" % (type(self).__name__, self.label)


class AccessNode(Node):
    def __init__(self, data: str):
        super().__init__(data)
        self.data = data


@dataclasses.dataclass
class Edge:
    src: Node
    src_conn: Optional[str]
    dst: Node
    dst_conn: Optional[str]
    data: Memlet


class SDFGState:
    def __init__(self, label: str, parent: "SDFG"):
        self.label = label
        self.parent = parent
        self._nodes: List[Node] = []
        self._edges: List[Edge] = []

    # -- construction
    def add_node(self, node: Node) -> Node:
        if node not in self._nodes:
            self._nodes.append(node)
        return node

    def add_access(self, name: str) -> AccessNode:
        if name not in self.parent.arrays:
            raise KeyError("array %r is not in the SDFG" % name)
        return self.add_node(AccessNode(name))

    add_read = add_access
    add_write = add_access

    def add_edge(self, src: Node, src_conn, dst: Node, dst_conn, memlet: Memlet) -> Edge:
        self.add_node(src)
        self.add_node(dst)
        if src_conn is not None and src_conn not in src.out_connectors:
            raise ValueError("%r has no output connector %r" % (src, src_conn))
        if dst_conn is not None and dst_conn not in dst.in_connectors:
            raise ValueError("%r has no input connector %r" % (dst, dst_conn))
        e = Edge(src, src_conn, dst, dst_conn, memlet)
        self._edges.append(e)
        return e

    def remove_node(self, node: Node):
        self._nodes.remove(node)
        self._edges = [e for e in self._edges if e.src is not node and e.dst is not node]

    def remove_edge(self, edge: Edge):
        self._edges.remove(edge)

    # -- queries
    def nodes(self) -> List[Node]:
        return list(self._nodes)

    def edges(self) -> List[Edge]:
        return list(self._edges)

    def in_edges(self, node: Node) -> List[Edge]:
        return [e for e in self._edges if e.dst is node]

    def out_edges(self, node: Node) -> List[Edge]:
        return [e for e in self._edges if e.src is node]

    def in_edges_by_connector(self, node: Node, conn: str) -> Iterable[Edge]:
        return (e for e in self._edges if e.dst is node and e.dst_conn == conn)

    def out_edges_by_connector(self, node: Node, conn: str) -> Iterable[Edge]:
        return (e for e in self._edges if e.src is node and e.src_conn == conn)

    def library_nodes(self) -> List[Node]:
        return [n for n in self._nodes if not isinstance(n, AccessNode)]

    def topological_sort(self) -> List[Node]:
        """Non-access nodes in an order where every producer of an array precedes its consumers
        (dependencies go through array names, so several access nodes of one array are fine)."""
        ops = self.library_nodes()
        arrays = self.parent.arrays

        def root(name):  # a view depends on whoever writes the buffer it aliases
            while name in arrays and arrays[name].view_of is not None:
                name = arrays[name].view_of
            return name

        writes = {id(n): {root(e.data.data) for e in self.out_edges(n)} for n in ops}
        reads = {id(n): {root(e.data.data) for e in self.in_edges(n)} for n in ops}
        producer = {}
        for n in ops:
            for a in writes[id(n)]:
                producer.setdefault(a, []).append(n)
        order, done, visiting = [], set(), set()

        def visit(n):
            if id(n) in done:
                return
            if id(n) in visiting:
                raise ValueError("cycle through %r" % n)
            visiting.add(id(n))
            for a in reads[id(n)]:
                for p in producer.get(a, []):
                    if p is not n:
                        visit(p)
            visiting.discard(id(n))
            done.add(id(n))
            order.append(n)

        for n in ops:
            visit(n)
        return order


class SDFG:
    def __init__(self, name: str):
        self.name = name
        self.arrays: Dict[str, Array] = {}
        self._states: List[SDFGState] = []
        self.constants: Dict[str, torch.Tensor] = {}
        #: Python values of scalar constants before rounding to the tensor dtype (an fp16 graph
        #: stores eps = 1e-12 as 0; the fused kernels take the exact value)
        self.constants_exact: Dict[str, float] = {}

    # -- data
    def add_datadesc(self, name: str, desc: Array, find_new_name: bool = False) -> str:
        if name in self.arrays:
            if not find_new_name:
                raise NameError("array %r already exists" % name)
            i = 0
            while "%s_%d" % (name, i) in self.arrays:
                i += 1
            name = "%s_%d" % (name, i)
        self.arrays[name] = desc
        return name

    def add_array(self, name, shape, dtype, transient=False, strides=None, find_new_name=False):
        name = self.add_datadesc(name, Array(shape, dtype, transient, strides), find_new_name)
        return name, self.arrays[name]

    def add_transient(self, name, shape, dtype, find_new_name=True):
        return self.add_array(name, shape, dtype, transient=True, find_new_name=find_new_name)

    def add_view(self, name, base: str, shape, strides, offset=0, find_new_name=True):
        root = self.arrays[base]
        while root.view_of is not None:
            offset += root.view_offset
            base = root.view_of
            root = self.arrays[base]
        desc = Array(shape, root.dtype, transient=True, strides=strides, view_of=base, view_offset=offset)
        name = self.add_datadesc(name, desc, find_new_name)
        return name, desc

    def add_constant(self, name: str, value: torch.Tensor):
        self.constants[name] = value

    def make_array_memlet(self, name: str) -> Memlet:
        if name not in self.arrays:
            raise KeyError(name)
        return Memlet(name)

    # -- states
    def add_state(self, label: Optional[str] = None) -> SDFGState:
        st = SDFGState(label or "state_%d" % len(self._states), self)
        self._states.append(st)
        return st

    def states(self) -> List[SDFGState]:
        return list(self._states)

    def node_id_label(self, node: Node) -> str:
        return node.label

    def arglist(self) -> Dict[str, Array]:
        """Non-transient arrays: what a caller has to pass (dace.SDFG.arglist)."""
        return {k: v for k, v in self.arrays.items() if not v.transient}

    def clone_desc(self, name: str) -> Array:
        return copy.deepcopy(self.arrays[name])


def in_desc_with_name(node: Node, state: SDFGState, sdfg: SDFG, name: str) -> Array:
    """daceml.util.utils.in_desc_with_name (daceml/util/utils.py:34-44)."""
    for e in state.in_edges_by_connector(node, name):
        return sdfg.arrays[e.data.data]
    raise KeyError("%r has no edge on input connector %r" % (node, name))


def out_desc_with_name(node: Node, state: SDFGState, sdfg: SDFG, name: str) -> Array:
    """daceml.util.utils.out_desc_with_name (daceml/util/utils.py:46-55)."""
    for e in state.out_edges_by_connector(node, name):
        return sdfg.arrays[e.data.data]
    raise KeyError("%r has no edge on output connector %r" % (node, name))


def in_edge_with_name(node, state, name) -> Edge:
    for e in state.in_edges_by_connector(node, name):
        return e
    raise KeyError("%r has no edge on input connector %r" % (node, name))


def out_edge_with_name(node, state, name) -> Edge:
    for e in state.out_edges_by_connector(node, name):
        return e
    raise KeyError("%r has no edge on output connector %r" % (node, name))
