"""Expansion and execution of SDFGs made of ONNX library nodes.

``expand_onnx_nodes`` is daceml.util.utils.expand_onnx_nodes (daceml/util/utils.py:156-203): every
``ONNXOp`` is replaced by the result of its selected implementation. ``CompiledSDFG`` is the stand-in
for DaCe's compiled SDFG plus DaCeML's ctypes dispatcher (daceml/torch/dispatchers/ctypes_module.py):
transients are owned by the SDFG and allocated once, caller arrays are passed per call, every kernel
is enqueued on the caller's current stream without synchronising (the ``nosync`` states of
ctypes_module.py:210-211).

Binding is done once: each launch becomes ``(ctypes function, tuple of ctypes arguments)``. Pointers of
caller-owned arrays live in shared mutable ``c_void_p`` objects that are updated on every call, so the
steady state is one ctypes call per kernel and no Python-side planning.
"""
import ctypes
import logging
from typing import Dict, List, Optional, Sequence

import torch

from . import _lib as L
from . import hip_tasklet as T
from . import memory_plan
from .onnx.nodes import ONNXOp
from .sdfg import SDFG, AccessNode, Array, SDFGState

log = logging.getLogger(__name__)

_ITEM = {torch.float16: 2, torch.float32: 4, torch.float64: 8, torch.int64: 8, torch.int32: 4, torch.bool: 1}


def expand_onnx_nodes(sdfg: SDFG, predicate=None) -> int:
    """Expand all ONNX library nodes (recursively: an expansion may return nodes that are themselves
    ONNX library nodes). Returns the number of expansions."""
    count = 0
    for state in sdfg.states():
        changed = True
        while changed:
            changed = False
            for node in state.nodes():
                if isinstance(node, ONNXOp) and (predicate is None or predicate(node)):
                    result = node.expand(sdfg, state)
                    _replace_node(state, node, result)
                    count += 1
                    changed = True
    return count


def _replace_node(state: SDFGState, node, new):
    for e in state.in_edges(node):
        if e.dst_conn not in new.in_connectors:
            raise ValueError("expansion of %r lacks input connector %r" % (node, e.dst_conn))
    for e in state.out_edges(node):
        if e.src_conn not in new.out_connectors:
            raise ValueError("expansion of %r lacks output connector %r" % (node, e.src_conn))
    state.add_node(new)
    for e in state.edges():
        if e.dst is node:
            e.dst = new
        if e.src is node:
            e.src = new
    state._nodes.remove(node)


def forwarded_transients(sdfg: SDFG, forward_states: Sequence[str], backward_states: Sequence[str]) -> List[str]:
    """Transient buffers that the forward states write and the backward states touch: the values a pending
    backward call depends on (what the reference's dispatcher turns into extra forward outputs and saves on the
    autograd context, daceml/autodiff/torch.py:56-104, ctypes_module.py:150-156)."""
    def root(name):
        while sdfg.arrays[name].view_of is not None:
            name = sdfg.arrays[name].view_of
        return name

    written, touched = set(), set()
    for state in sdfg.states():
        for e in state.edges():
            r = root(e.data.data)
            if state.label in forward_states and isinstance(e.dst, AccessNode):
                written.add(r)
            if state.label in backward_states:
                touched.add(r)
    return [n for n, d in sdfg.arrays.items() if n in written and n in touched and d.transient and d.view_of is None
            and n not in sdfg.constants]


class _Launch:
    __slots__ = ("fn", "args", "label", "symbol", "flops", "bytes_moved", "kind", "state")

    def __init__(self, fn, args, label, symbol, flops, bytes_moved, kind, state):
        self.fn, self.args, self.label, self.symbol = fn, args, label, symbol
        self.flops, self.bytes_moved, self.kind, self.state = flops, bytes_moved, kind, state


class CapturedLaunches:
    """A HIP graph of a CompiledSDFG's launches under one binding (``CompiledSDFG.capture``)."""
    def __init__(self, program: "CompiledSDFG", graph, binding: int):
        self.program, self.graph, self.binding = program, graph, binding

    def replay(self):
        """Enqueue the recorded launches on the current stream."""
        if self.program._binding != self.binding:
            raise RuntimeError("the program has been bound to other tensors since this graph was captured; capture again")
        self.graph.replay()


class CompiledSDFG:
    """An expanded SDFG bound to device buffers; call it with the non-transient arrays by name."""
    def __init__(self, sdfg: SDFG, device: Optional[torch.device] = None, expand: bool = True,
                 reuse_transients: bool = False, outside_arena: Sequence[str] = ()):
        """``reuse_transients``: transients whose lifetimes (first to last node that touches them, in launch order over
        all states) do not overlap share memory inside one arena, a buffer that dies handing its bytes to the next
        one that is born. The step then touches fewer distinct bytes between two uses of the same tensor, which is
        what decides whether the second use finds it in the 256 MB last-level cache. Off by default: after a run the
        transients of such a program no longer all hold their values (``buffers[name]`` of a dead one shows whatever
        was written over it)."""
        self.sdfg = sdfg
        self.reuse_transients = bool(reuse_transients)
        #: transients that keep a buffer of their own (a caller that rebinds them to its own memory on every call
        #: would leave their place in the arena unused)
        self.outside_arena = tuple(outside_arena)
        self.arena_bytes = 0
        self.device = torch.device(device) if device is not None else torch.device("cuda", torch.cuda.current_device())
        if self.device.type != "cuda":
            raise ValueError("the HIP implementations run on a GPU device; got %s" % self.device)
        self.lib = L.load()
        if expand:
            expand_onnx_nodes(sdfg)
        self._keep = []                       # ctypes objects that must outlive the launches
        self._ptr: Dict[str, ctypes.c_void_p] = {}
        self._derived = []                    # (c_void_p, base name, byte offset)
        self._ptr_arrays = []                 # (ctypes array, [(slot, name)])
        self._stream = ctypes.c_void_p(0)
        self._binding = 0                     # bumped whenever a pointer may have changed
        self.buffers: Dict[str, torch.Tensor] = {}
        # [(state, node)]: the order the kernels are enqueued in
        self._order = memory_plan.launch_order(sdfg, small_peak=self.reuse_transients)
        self._allocate()
        self._launches: List[_Launch] = []
        ws = 0
        for state, node in self._order:
            if isinstance(node, ONNXOp):
                raise RuntimeError("unexpanded library node %r" % node)
            ws = max(ws, getattr(node, "workspace_bytes", 0))
        self._ws_bytes = max(int(ws), 256)
        self._workspace = torch.empty(self._ws_bytes, dtype=torch.uint8, device=self.device)
        for state, node in self._order:
            self._bind_node(state, node)
        self._refresh()

    # -- memory ------------------------------------------------------------
    def _allocate(self):
        for name, desc in self.sdfg.arrays.items():
            self._ptr[name] = ctypes.c_void_p(0)
        for name, desc in self.sdfg.arrays.items():
            if desc.view_of is not None:
                self._derived.append((self._ptr[name], desc.view_of, desc.view_offset * _ITEM[desc.dtype]))
            elif name in self.sdfg.constants:
                t = self.sdfg.constants[name].to(device=self.device, dtype=desc.dtype).contiguous()
                if tuple(t.shape) != desc.shape:
                    raise ValueError("constant %r has shape %s, descriptor says %s" % (name, tuple(t.shape), desc.shape))
                self.buffers[name] = t
            elif desc.transient:
                self.buffers[name] = None     # placed below
        plan = memory_plan.place_transients(self.sdfg, self._order, leave_out=self.outside_arena) \
            if self.reuse_transients else {}
        if plan:
            self.arena_bytes = max(off + memory_plan.nbytes(self.sdfg.arrays[name]) for name, off in plan.items())
            self._arena = torch.empty(self.arena_bytes, dtype=torch.uint8, device=self.device)
        for name in [n for n, t in self.buffers.items() if t is None]:
            desc = self.sdfg.arrays[name]
            if name in plan:
                piece = self._arena[plan[name]:plan[name] + memory_plan.nbytes(desc)]
                self.buffers[name] = piece.view(desc.dtype).view(desc.shape)
            else:
                self.buffers[name] = torch.empty(desc.shape, dtype=desc.dtype, device=self.device)
        for name, t in self.buffers.items():
            self._ptr[name].value = t.data_ptr()

    def _refresh(self, changed: bool = True):
        if changed:
            self._binding += 1
        for obj, base, off in self._derived:
            obj.value = (self._ptr[base].value or 0) + off
        for arr, slots in self._ptr_arrays:
            for i, name in slots:
                arr[i] = self._ptr[name].value

    # -- binding -----------------------------------------------------------
    def _bind_node(self, state: SDFGState, node):
        calls = getattr(node, "calls", None)
        if calls is None:
            if isinstance(node, AccessNode):
                return
            raise RuntimeError("node %r has no HIP calls; only HipTasklet / ViewTasklet nodes can run" % node)
        conn_to_array = {}
        for e in state.in_edges(node):
            conn_to_array[e.dst_conn] = e.data.data
        for e in state.out_edges(node):
            conn_to_array[e.src_conn] = e.data.data
        for call in calls:
            fn = getattr(self.lib, call.symbol)
            args = []
            for a in call.args:
                if isinstance(a, T.Ptr):
                    name = conn_to_array[a.conn]
                    if a.offset:
                        obj = ctypes.c_void_p(0)
                        self._derived.append((obj, name, a.offset * _ITEM[self.sdfg.arrays[name].dtype]))
                        args.append(obj)
                    else:
                        args.append(self._ptr[name])
                elif isinstance(a, T.Null):
                    # None, not c_void_p(0): for a POINTER(c_void_p) parameter ctypes would pass the ADDRESS of a
                    # c_void_p instance (a non-NULL pointer table with one NULL entry)
                    args.append(None)
                elif isinstance(a, T.I64):
                    args.append(ctypes.c_int64(a.value))
                elif isinstance(a, T.I32):
                    args.append(ctypes.c_int(a.value))
                elif isinstance(a, T.F32):
                    args.append(ctypes.c_float(a.value))
                elif isinstance(a, T.USize):
                    args.append(ctypes.c_size_t(a.value))
                elif isinstance(a, T.I64Array):
                    arr = (ctypes.c_int64 * max(len(a.values), 1))(*a.values)
                    self._keep.append(arr)
                    args.append(arr)
                elif isinstance(a, T.PtrArray):
                    arr = (ctypes.c_void_p * len(a.conns))()
                    self._ptr_arrays.append((arr, [(i, conn_to_array[c]) for i, c in enumerate(a.conns)]))
                    args.append(arr)
                elif isinstance(a, T.Struct):
                    self._keep.append(a.value)
                    args.append(ctypes.byref(a.value))
                elif isinstance(a, T.Workspace):
                    args.append(ctypes.c_void_p(self._workspace.data_ptr() + a.offset))
                elif isinstance(a, T.WorkspaceBytes):
                    args.append(ctypes.c_size_t(self._ws_bytes - a.offset))
                elif isinstance(a, T.Stream):
                    args.append(self._stream)
                else:
                    raise TypeError("unknown HIP call argument %r" % (a, ))
            # work is attributed to the node's first call only (later calls are follow-up passes)
            first = call is calls[0]
            flops = call.flops if call.flops is not None else (node.flops if first else 0)
            moved = call.bytes_moved if call.bytes_moved is not None else (node.bytes_moved if first else 0)
            self._launches.append(_Launch(fn, tuple(args), node.label, call.symbol, flops, moved, node.kind, state.label))

    # -- execution -----------------------------------------------------------
    def _bind_arguments(self, kwargs: Dict[str, torch.Tensor], partial: bool = False):
        changed = False
        for name, desc in self.sdfg.arrays.items():
            if desc.transient or name in self.sdfg.constants or desc.view_of is not None:
                continue
            if name not in kwargs:
                if partial:
                    continue
                raise TypeError("missing argument %r (arrays to pass: %s)" % (name, sorted(self.arglist())))
            t = kwargs[name]
            if not isinstance(t, torch.Tensor) or t.device != self.device:
                raise ValueError("argument %r must be a tensor on %s" % (name, self.device))
            if t.dtype != desc.dtype or tuple(t.shape) != desc.shape:
                raise ValueError("argument %r: expected %s %s, got %s %s" % (name, desc.dtype, desc.shape, t.dtype,
                                                                             tuple(t.shape)))
            if tuple(t.stride()) != desc.strides and t.numel() > 1:
                raise ValueError("argument %r must have strides %s (pass a contiguous tensor)" % (name, desc.strides))
            if self._ptr[name].value != t.data_ptr():
                changed = True
            self._ptr[name].value = t.data_ptr()
        extra = set(kwargs) - set(self.sdfg.arrays)
        if extra:
            raise TypeError("unknown argument(s) %s" % sorted(extra))
        self._refresh(changed)

    def arglist(self) -> Dict[str, Array]:
        return {k: v for k, v in self.sdfg.arrays.items()
                if not v.transient and k not in self.sdfg.constants and v.view_of is None}

    def __call__(self, **kwargs):
        self._bind_arguments(kwargs)
        self.launch()

    def bind(self, tensors: Dict[str, torch.Tensor]):
        """Bind some of the caller-owned arrays; the others keep the pointers of their last binding. For callers
        that run the states separately (forward now, backward later) with ``launch(states)``; the tensors must stay
        alive until the launches that use them have been enqueued."""
        self._bind_arguments(tensors, partial=True)

    def forwarded_transients(self, forward_states: Sequence[str], backward_states: Sequence[str]) -> List[str]:
        """See the module-level function."""
        return forwarded_transients(self.sdfg, forward_states, backward_states)

    def rebind_transients(self, tensors: Dict[str, torch.Tensor], release: bool = False):
        """Point transient arrays at caller-provided buffers (same shape and dtype, dense). With ``release`` the
        buffers this object allocated for them are dropped."""
        for name, t in tensors.items():
            desc = self.sdfg.arrays[name]
            if not desc.transient or desc.view_of is not None or name in self.sdfg.constants:
                raise ValueError("%r is not a transient buffer of this SDFG" % name)
            if t.dtype != desc.dtype or tuple(t.shape) != desc.shape or not t.is_contiguous() or t.device != self.device:
                raise ValueError("buffer for %r must be a dense %s %s tensor on %s" % (name, desc.dtype, desc.shape,
                                                                                        self.device))
            self._ptr[name].value = t.data_ptr()
            if release:
                self.buffers[name] = t
        self._refresh()

    def launch(self, states: Optional[Sequence[str]] = None):
        """Enqueue every kernel (of the named states) on the current stream, with the pointers of the
        last binding."""
        self._stream.value = torch.cuda.current_stream(self.device).cuda_stream
        for l in self._launches:
            if states is not None and l.state not in states:
                continue
            status = l.fn(*l.args)
            if status != 0:
                raise L.HipKernelError(status, "%s (%s): %s" % (l.label, l.symbol, L.last_error()))

    def capture(self, states: Optional[Sequence[str]] = None, warmup: int = 2) -> "CapturedLaunches":
        """The launches (of the named states) with the pointers of the current binding, recorded once into a HIP graph:
        ``replay()`` then costs one graph launch instead of one host call per kernel, which is what a step of a few
        short kernels is bound by. The library allocates nothing, copies nothing and clears nothing on the host side
        of a call, so every entry point can be recorded. The graph holds raw pointers: it belongs to the binding it
        was captured under and refuses to replay after ``bind`` / ``__call__`` / ``rebind_transients`` changed it."""
        current = torch.cuda.current_stream(self.device)
        side = torch.cuda.Stream(self.device)
        side.wait_stream(current)
        with torch.cuda.stream(side):
            for _ in range(max(warmup, 1)):   # first launches set kernel attributes (large LDS) outside the capture
                self.launch(states)
        current.wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            self.launch(states)
        return CapturedLaunches(self, graph, self._binding)

    def launch_timed(self):
        """Like launch(), with one HIP event on the launch stream before the first kernel and one after every kernel;
        returns [(launch, ms)] where a launch's time runs from the event before it to the event after it - the kernel
        and its dispatch on the stream. The times add up to the time of the whole sequence between the first and the
        last event."""
        self._stream.value = torch.cuda.current_stream(self.device).cuda_stream
        marks = [torch.cuda.Event(enable_timing=True)]
        marks[0].record()
        for l in self._launches:
            status = l.fn(*l.args)
            e = torch.cuda.Event(enable_timing=True)
            e.record()
            marks.append(e)
            if status != 0:
                raise L.HipKernelError(status, "%s (%s): %s" % (l.label, l.symbol, L.last_error()))
        torch.cuda.synchronize(self.device)
        return [(l, marks[i].elapsed_time(marks[i + 1])) for i, l in enumerate(self._launches)]

    @property
    def launches(self) -> Sequence[_Launch]:
        return tuple(self._launches)
