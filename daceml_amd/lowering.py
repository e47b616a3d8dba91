"""Expanded library nodes as C++ source.

A "hip" expansion is a list of C-ABI calls (``hip_tasklet.HipCall``). This module renders such calls as the body
of a C++ tasklet - what the reference's native expansions return (the cuDNN tasklets of
daceml/onnx/op_implementations/cudnn_implementations.py:360-410, built on ``empty_sdfg_for_node``,
daceml/onnx/op_implementations/utils.py:105-139) - and lowers a whole expanded state to a ``TaskletProgram``:
arrays plus an ordered list of tasklets with pointer connectors. Two consumers:

* ``daceml_amd.dace_plugin`` turns a ``TaskletProgram`` into a nested ``dace.SDFG`` of C++ tasklets (the form in
  which forward expansions, reverse nodes and fused states reach a real DaCeML);
* ``emit_cxx`` writes the program as one freestanding ``extern "C"`` function over ``include/daceml_hip.h`` - the
  ahead-of-time form of what ``runtime.CompiledSDFG`` does through ctypes, and what the host-side tests compile to
  pin every rendered call against the header's declarations.
"""
import dataclasses
from typing import Callable, Dict, List, Optional, Tuple

import torch

from . import hip_tasklet as T
from .sdfg import SDFG, AccessNode, Array, SDFGState

#: element type names in generated code; ``half`` stands for whatever 2-byte type the consumer declares
CXX_TYPES = {torch.float16: "half", torch.float32: "float", torch.float64: "double", torch.int64: "int64_t",
             torch.int32: "int32_t", torch.bool: "bool", torch.uint8: "uint8_t"}


def _float_literal(v: float) -> str:
    v = float(v)
    if v != v:
        return "NAN"
    if v in (float("inf"), float("-inf")):
        return "INFINITY" if v > 0 else "-INFINITY"
    return "%.9ef" % v


def render_calls(calls: List[T.HipCall], conn_expr: Callable[[str, int], str], on_error: str,
                 workspace: str = "__state->dmlhip_workspace", workspace_bytes: str = "__state->dmlhip_workspace_bytes",
                 stream: str = "(void*)__dace_current_stream") -> str:
    """C++ statements that perform `calls`. ``conn_expr(connector, element offset)`` is the pointer expression of a
    connector; ``on_error`` is a statement template run when a call returns non-zero (``{symbol}`` and ``{status}``
    are substituted). Index arrays, pointer tables and descriptor structs become locals declared ahead of the call
    that uses them."""
    lines, n = [], 0
    for call in calls:
        args = []
        for a in call.args:
            if isinstance(a, T.Ptr):
                args.append(conn_expr(a.conn, a.offset))
            elif isinstance(a, T.Null):
                args.append("nullptr")
            elif isinstance(a, (T.I64, T.I32, T.USize)):
                args.append(str(int(a.value)))
            elif isinstance(a, T.F32):
                args.append(_float_literal(a.value))
            elif isinstance(a, T.Stream):
                args.append(stream)
            elif isinstance(a, T.I64Array):
                name = "__dml_arr%d" % n
                n += 1
                lines.append("const int64_t %s[] = {%s};" % (name, ", ".join(str(int(v)) for v in a.values) or "0"))
                args.append(name)
            elif isinstance(a, T.PtrArray):
                name = "__dml_ptrs%d" % n
                n += 1
                # void*[]: converts to both `const void* const*` (inputs) and `void* const*` (outputs)
                lines.append("void* %s[] = {%s};" % (name, ", ".join("(void*)" + conn_expr(c, 0) for c in a.conns)))
                args.append(name)
            elif isinstance(a, T.Struct):
                name = "__dml_desc%d" % n
                n += 1
                fields = []
                for fname, ftype in a.value._fields_:
                    v = getattr(a.value, fname)
                    if hasattr(v, "__len__"):
                        fields.append("{%s}" % ", ".join(str(int(x)) for x in v))
                    elif "float" in str(ftype):
                        fields.append(_float_literal(v))
                    else:
                        fields.append(str(int(v)))
                lines.append("%s %s = {%s};" % (a.c_type, name, ", ".join(fields)))
                args.append("&" + name)
            elif isinstance(a, T.Workspace):
                args.append("((char*)%s + %d)" % (workspace, a.offset) if a.offset else "(void*)%s" % workspace)
            elif isinstance(a, T.WorkspaceBytes):
                args.append("(size_t)(%s - %d)" % (workspace_bytes, a.offset) if a.offset else
                            "(size_t)%s" % workspace_bytes)
            else:
                raise NotImplementedError("no C++ rendering for argument %r" % (a, ))
        lines.append("if (int __dml_status = %s(%s)) { %s }" %
                     (call.symbol, ", ".join(args), on_error.format(symbol=call.symbol, status="__dml_status")))
    return "\n".join(lines)


#: what a DaCe tasklet does when a call fails: report and unwind (the reference's ORT path prints and exits,
#: daceml/onnx/include/dace_onnx.h:7-15; its cuDNN path prints and goes on, daceml_cudnn.h:15-22)
TASKLET_ON_ERROR = ('throw std::runtime_error(std::string("{symbol} failed with status ") + std::to_string({status}) + '
                    '": " + dmlhip_last_error_string());')


def render_tasklet_code(tasklet: T.HipTasklet, conn_ptr: Optional[Callable[[str], str]] = None) -> str:
    """C++ body of a DaCe tasklet performing the calls of `tasklet`; connector ``X`` is the pointer ``_X``."""
    conn_ptr = conn_ptr or (lambda c: "_" + c)
    return render_calls(tasklet.calls, lambda c, off: "(%s + %d)" % (conn_ptr(c), off) if off else conn_ptr(c),
                        TASKLET_ON_ERROR)


# ----------------------------------------------------------------------------- whole states
@dataclasses.dataclass
class TaskletSpec:
    """One C++ tasklet: pointer connectors ``_<connector>`` attached to whole arrays."""
    label: str
    inputs: Dict[str, str]       # connector -> array
    outputs: Dict[str, str]      # connector -> array
    calls: List[T.HipCall]
    offsets: Dict[str, int]      # connector -> element offset into its array (views, slices)

    def code(self, on_error: str = TASKLET_ON_ERROR, **names) -> str:
        def expr(conn, off):
            off += self.offsets.get(conn, 0)
            return "(_%s + %d)" % (conn, off) if off else "_" + conn
        return render_calls(self.calls, expr, on_error, **names)


@dataclasses.dataclass
class TaskletProgram:
    """An expanded state: the arrays it touches (views resolved to the arrays they alias) and its tasklets in
    execution order."""
    name: str
    arrays: Dict[str, Array]
    constants: Dict[str, torch.Tensor]
    tasklets: List[TaskletSpec]
    workspace_bytes: int

    def arguments(self) -> List[str]:
        """Arrays the caller provides, in declaration order (constants included: their values are the caller's to
        upload, as DaCeML's importer does with ``ONNXModel.weights``)."""
        return [n for n, d in self.arrays.items() if not d.transient]

    def transients(self) -> List[str]:
        return [n for n, d in self.arrays.items() if d.transient]


def _resolve(sdfg: SDFG, name: str) -> Tuple[str, int]:
    off = 0
    while sdfg.arrays[name].view_of is not None:
        off += sdfg.arrays[name].view_offset
        name = sdfg.arrays[name].view_of
    return name, off


def lower_state(sdfg: SDFG, state: SDFGState, name: Optional[str] = None) -> TaskletProgram:
    """Lower an expanded state (HipTasklet / ViewTasklet / access nodes only) to a TaskletProgram."""
    used: Dict[str, Array] = {}
    tasklets: List[TaskletSpec] = []
    ws = 0
    for node in state.topological_sort():
        calls = getattr(node, "calls", None)
        if calls is None:
            raise ValueError("state %r holds %r, which is not an expanded node (run expand_onnx_nodes first)" %
                             (state.label, node))
        if not calls:
            continue   # a view: its consumers address the aliased array directly
        ins, outs, offsets = {}, {}, {}
        for edges, table, conn_of in ((state.in_edges(node), ins, lambda e: e.dst_conn),
                                      (state.out_edges(node), outs, lambda e: e.src_conn)):
            for e in edges:
                root, off = _resolve(sdfg, e.data.data)
                conn = conn_of(e)
                if conn in ins or conn in outs:
                    raise ValueError("%r: connector %r is attached twice" % (node, conn))
                table[conn] = root
                if off:
                    offsets[conn] = off
                used.setdefault(root, sdfg.arrays[root])
        tasklets.append(TaskletSpec(node.label, ins, outs, list(calls), offsets))
        ws = max(ws, int(getattr(node, "workspace_bytes", 0)))
    # arrays in the SDFG's own order, so that the argument list is stable
    arrays = {n: d for n, d in sdfg.arrays.items() if n in used}
    constants = {n: t for n, t in sdfg.constants.items() if n in arrays}
    return TaskletProgram(name or "%s_%s" % (sdfg.name, state.label), arrays, constants, tasklets, ws)


# ----------------------------------------------------------------------------- freestanding C++
CXX_PRELUDE = """#include <stddef.h>
#include <stdint.h>
#include <math.h>
#include "daceml_hip.h"
#ifndef DMLHIP_HALF_DEFINED
#define DMLHIP_HALF_DEFINED
typedef struct { uint16_t bits; } half;   /* storage only: the library does the arithmetic */
#endif
"""


def emit_cxx(program: TaskletProgram, function: Optional[str] = None, prelude: bool = True) -> str:
    """The program as ``extern "C" int <function>(void* const* arguments, void* const* transients, void* workspace,
    size_t workspace_bytes, void* stream)``: ``arguments`` in the order of ``program.arguments()``, ``transients`` in
    the order of ``program.transients()`` (buffers of the arrays' sizes, owned by the caller), one workspace of at
    least ``program.workspace_bytes`` bytes. Enqueues every kernel on `stream` and returns 0, or the first non-zero
    status (``dmlhip_last_error_string()`` has the text)."""
    function = function or "dmlhip_program_" + "".join(c if c.isalnum() else "_" for c in program.name)
    out = [CXX_PRELUDE] if prelude else []
    out.append('extern "C" int %s(void* const* arguments, void* const* transients, void* workspace, '
               'size_t workspace_bytes, void* stream) {' % function)
    out.append("    if (workspace_bytes < %du) return DMLHIP_ERR_WORKSPACE;" % program.workspace_bytes)
    index = {n: ("arguments", i) for i, n in enumerate(program.arguments())}
    index.update({n: ("transients", i) for i, n in enumerate(program.transients())})
    for i, t in enumerate(program.tasklets):
        out.append("    {   // %s" % t.label)
        for conn, arr in list(t.inputs.items()) + list(t.outputs.items()):
            table, slot = index[arr]
            ctype = CXX_TYPES[program.arrays[arr].dtype]
            out.append("        %s* _%s = (%s*)%s[%d];   // %s" % (ctype, conn, ctype, table, slot, arr))
        body = t.code(on_error="return {status};", workspace="workspace", workspace_bytes="workspace_bytes",
                      stream="stream")
        out.extend("        " + line for line in body.splitlines())
        out.append("    }")
    out.append("    return 0;")
    out.append("}")
    return "\n".join(out) + "\n"


# ----------------------------------------------------------------------------- reverse nodes
@dataclasses.dataclass
class LoweredBackward:
    """The reverse of one forward node as a TaskletProgram whose arrays carry connector names: forward inputs and
    outputs it reads are named after the forward node's connectors, gradients after the connectors of
    ``BackwardResult`` - the naming contract of daceml/autodiff/base_abc.py:75-108."""
    program: TaskletProgram
    given_grad_names: Dict[str, str]       # forward output connector -> array holding its gradient (an input)
    required_grad_names: Dict[str, str]    # forward input connector -> array receiving its gradient (an output)
    forward_inputs: List[str]              # forward input connectors whose arrays the program reads
    forward_outputs: List[str]             # forward output connectors whose arrays the program reads


def lower_backward(node, state: SDFGState, sdfg: SDFG, impl, given: List[str], required: List[str]) -> LoweredBackward:
    """Run the backward implementation `impl` for `node` (a library node of `state` in `sdfg`, both of which are
    modified: pass copies), expand what it adds with the selected implementations and lower it. Raises
    ``NotApplicable`` when the reverse needs something a stand-alone reverse node cannot have (extra outputs of the
    forward node, such as LayerNormalization's statistics)."""
    from .autodiff.base_abc import BackwardContext, BackwardGroup
    from .onnx.nodes import NotApplicable, ONNXOp
    from . import onnx as donnx
    bstate = sdfg.add_state(node.label + "_reverse")
    ctx = BackwardContext(sdfg, state, sdfg, bstate, None)
    outs_before = set(node.out_connectors)
    rev, result = impl.backward(node, ctx, list(given), list(required))
    if set(node.out_connectors) != outs_before:
        raise NotApplicable("%r: the reverse node needs outputs the forward node does not have: %s" %
                            (node, sorted(set(node.out_connectors) - outs_before)))

    def fwd_array(conn, out):
        edges = state.out_edges_by_connector(node, conn) if out else state.in_edges_by_connector(node, conn)
        return next(iter(edges)).data.data

    def fresh(name):
        base, i = name, 0
        while name in sdfg.arrays:
            i += 1
            name = "%s_%d" % (base, i)
        return name

    given_names, required_names = {}, {}
    for conn in given:
        gconn = result.given_grad_names.get(conn)
        if gconn is None:
            continue
        d = sdfg.arrays[fwd_array(conn, True)]
        name = fresh(gconn)
        sdfg.add_array(name, d.shape, d.dtype)
        given_names[conn] = name
        targets = rev.inputs.get(gconn, []) if isinstance(rev, BackwardGroup) else [(rev, gconn)]
        for tgt, tconn in targets:
            bstate.add_edge(bstate.add_read(name), None, tgt, tconn, sdfg.make_array_memlet(name))
    for conn in required:
        d = sdfg.arrays[fwd_array(conn, False)]
        if conn in result.passthrough:
            # the gradient of this input IS the gradient given for an output (a residual Add): a stand-alone
            # reverse node has to hand it out as an array of its own
            src = given_names[result.passthrough[conn]]
            name = fresh(conn + "_grad")
            sdfg.add_array(name, d.shape, d.dtype)
            ident = donnx.ONNXIdentity("%s_%s_grad_copy" % (node.label, conn))
            bstate.add_edge(bstate.add_read(src), None, ident, "input", sdfg.make_array_memlet(src))
            bstate.add_edge(ident, "output", bstate.add_write(name), None, sdfg.make_array_memlet(name))
        else:
            gconn = result.required_grad_names.get(conn)
            if gconn is None:
                raise NotApplicable("%r: no gradient is computed for input %r" % (node, conn))
            name = fresh(gconn)
            sdfg.add_array(name, d.shape, d.dtype)
            src, sconn = rev.outputs[gconn] if isinstance(rev, BackwardGroup) else (rev, gconn)
            bstate.add_edge(src, sconn, bstate.add_write(name), None, sdfg.make_array_memlet(name))
        required_names[conn] = name

    changed = True
    while changed:   # expansions may return library nodes that expand further
        changed = False
        for n in bstate.nodes():
            if isinstance(n, ONNXOp):
                new = n.expand(sdfg, bstate)
                for e in bstate.edges():
                    if e.dst is n:
                        e.dst = new
                    if e.src is n:
                        e.src = new
                bstate.add_node(new)
                bstate._nodes.remove(n)
                changed = True
    program = lower_state(sdfg, bstate, name=node.label + "_backward")

    # name the forward arrays after the forward node's connectors
    rename, fwd_in, fwd_out = {}, [], []
    grads = set(given_names.values()) | set(required_names.values())
    for e in state.in_edges(node):
        root, _ = _resolve(sdfg, e.data.data)
        if root in program.arrays and root not in grads and root not in rename:
            rename[root] = e.dst_conn
            fwd_in.append(e.dst_conn)
    for e in state.out_edges(node):
        root, _ = _resolve(sdfg, e.data.data)
        if root in program.arrays and root not in grads and root not in rename:
            rename[root] = e.src_conn
            fwd_out.append(e.src_conn)
    foreign = [a for a in program.arguments() if a not in rename and a not in grads and a not in program.constants]
    if foreign:
        raise NotApplicable("%r: the reverse node reads arrays that are not connected to the forward node: %s" %
                            (node, foreign))
    taken = set(program.arrays) - set(rename)
    for old, new in list(rename.items()):
        if new in taken:
            raise NotApplicable("%r: connector name %r collides with an array of the reverse node" % (node, new))
    program = rename_arrays(program, rename)
    # whatever the forward graph holds them in, to the reverse node its forward values are inputs
    import copy
    for name in rename.values():
        d = copy.copy(program.arrays[name])
        d.transient = False
        program.arrays[name] = d
    return LoweredBackward(program, given_names, required_names, fwd_in, fwd_out)


def rename_arrays(program: TaskletProgram, rename: Dict[str, str]) -> TaskletProgram:
    r = lambda a: rename.get(a, a)  # noqa: E731
    return TaskletProgram(
        program.name, {r(n): d for n, d in program.arrays.items()}, {r(n): t for n, t in program.constants.items()},
        [TaskletSpec(t.label, {c: r(a) for c, a in t.inputs.items()}, {c: r(a) for c, a in t.outputs.items()},
                     t.calls, t.offsets) for t in program.tasklets], program.workspace_bytes)
