"""Registers the "hip" implementations inside a real DaCeML installation.

Only meaningful where ``dace`` and ``daceml`` import (neither does in the build image, so this module
has not been executed; it is kept small and follows the cuDNN expansion,
daceml/onnx/op_implementations/cudnn_implementations.py:123-410, and its environment,
daceml/onnx/environments/cudnn.py:11-70, line by line).

``install()``:
  1. defines a ``@dace.library.environment`` that adds ``include/`` and links ``libdaceml_hip.so``;
  2. for every implementation in this package's ``ONNXForward`` registry builds a DaCeML ``ONNXForward``
     subclass whose ``forward`` runs this package's planner on descriptors taken from the DaCe SDFG and
     renders the resulting ``HipCall``s as the body of a C++ tasklet with pointer connectors;
  3. registers it twice — ``@op_implementation`` (so autodiff's registry lookups see it) and
     ``donnx.ONNX<Op>.register_implementation`` wrapped like onnx_op.py:668-697 (node classes snapshot
     the registry at import time, so the decorator alone is not enough);
  4. registers the ``BackwardImplementation``s the same way.
After ``install()``, ``donnx.default_implementation = "hip"`` (or ``node.implementation = "hip"``) selects
the kernels for existing SDFGs, the PyTorch frontend and autodiff-generated nodes.
"""
import os

from . import hip_tasklet as T
from . import _lib as L

_ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _c_literal(arg, conn_ptr):
    """C++ expression for one HipCall argument; `conn_ptr` maps a connector to its tasklet pointer name."""
    if isinstance(arg, T.Ptr):
        return "(%s + %d)" % (conn_ptr(arg.conn), arg.offset) if arg.offset else conn_ptr(arg.conn)
    if isinstance(arg, T.Null):
        return "nullptr"
    if isinstance(arg, (T.I64, T.I32, T.USize)):
        return str(int(arg.value))
    if isinstance(arg, T.F32):
        return "%.9ef" % arg.value
    if isinstance(arg, T.Stream):
        return "(void*)__dace_current_stream"
    raise NotImplementedError(type(arg).__name__)


def render_tasklet_code(tasklet: T.HipTasklet, conn_ptr=lambda c: "_" + c):
    """C++ body of a DaCe tasklet that performs the tasklet's HipCalls. Arrays, descriptor structs and the
    workspace become locals / state fields declared ahead of the calls."""
    lines, n = [], 0
    for call in tasklet.calls:
        args = []
        for a in call.args:
            if isinstance(a, T.I64Array):
                name = "__dml_arr%d" % n
                n += 1
                lines.append("const int64_t %s[] = {%s};" % (name, ", ".join(str(int(v)) for v in a.values) or "0"))
                args.append(name)
            elif isinstance(a, T.PtrArray):
                name = "__dml_ptrs%d" % n
                n += 1
                # void*[]: converts to both `const void* const*` (inputs) and `void* const*` (outputs)
                lines.append("void* %s[] = {%s};" % (name, ", ".join("(void*)" + conn_ptr(c) for c in a.conns)))
                args.append(name)
            elif isinstance(a, T.Struct):
                name = "__dml_desc%d" % n
                n += 1
                fields = []
                for fname, ftype in a.value._fields_:
                    v = getattr(a.value, fname)
                    if hasattr(v, "__len__"):
                        fields.append("{%s}" % ", ".join(str(x) for x in v))
                    else:
                        fields.append(repr(float(v)) + "f" if "float" in str(ftype) else str(int(v)))
                lines.append("%s %s = {%s};" % (a.c_type, name, ", ".join(fields)))
                args.append("&" + name)
            elif isinstance(a, T.Workspace):
                args.append("((char*)__state->dmlhip_workspace + %d)" % a.offset)
            elif isinstance(a, T.WorkspaceBytes):
                args.append("(__state->dmlhip_workspace_bytes - %d)" % a.offset)
            else:
                args.append(_c_literal(a, conn_ptr))
        lines.append('if (int __s = %s(%s)) { fprintf(stderr, "%s: %%s\\n", dmlhip_last_error_string()); }' %
                     (call.symbol, ", ".join(args), call.symbol))
    return "\n".join(lines)


def install():
    """Register everything with an importable DaCeML. Raises ImportError where dace / daceml are absent."""
    import dace
    import dace.library
    from dace import nodes as dnodes
    from dace.transformation.transformation import ExpandTransformation
    import daceml.onnx as donnx
    from daceml.onnx.forward_implementation_abc import ONNXForward as RefONNXForward
    from daceml.onnx.op_implementations.utils import op_implementation as ref_op_implementation
    from daceml.util.utils import in_desc_with_name, out_desc_with_name  # noqa: F401

    from . import onnx as our_onnx
    from .onnx.forward_implementation_abc import ONNXForward as OurONNXForward
    from .sdfg import SDFG as OurSDFG, Array as OurArray

    lib_dir = os.path.join(_ROOT, "daceml_amd", "csrc")

    @dace.library.environment
    class DaceMLHip:
        """Links libdaceml_hip.so (pattern: daceml/onnx/environments/cudnn.py:11-49)."""
        cmake_minimum_version = None
        cmake_packages = []
        cmake_variables = {}
        cmake_includes = [os.path.join(_ROOT, "include")]
        cmake_libraries = [os.path.join(lib_dir, "libdaceml_hip.so")]
        cmake_compile_flags = []
        cmake_link_flags = ["-L" + lib_dir, "-Wl,-rpath," + lib_dir]
        cmake_files = []
        state_fields = ["void* dmlhip_workspace;", "size_t dmlhip_workspace_bytes;"]
        headers = ["daceml_hip.h", "cstdio"]
        init_code = ("__state->dmlhip_workspace_bytes = 256u << 20;\n"
                     "hipMalloc(&__state->dmlhip_workspace, __state->dmlhip_workspace_bytes);")
        finalize_code = "hipFree(__state->dmlhip_workspace);"
        dependencies = []

    import torch
    _to_torch = {dace.float16: torch.float16, dace.float32: torch.float32, dace.float64: torch.float64,
                 dace.int64: torch.int64, dace.int32: torch.int32, dace.bool: torch.bool}

    def mirror(node, state, sdfg):
        """Rebuild the node with this package's classes on a one-node stand-in SDFG (descriptors only)."""
        s = OurSDFG(node.label)
        st = s.add_state()
        attrs = {a: getattr(node, a) for a in our_onnx.get_onnx_node(node.schema.name).schema.attributes
                 if hasattr(node, a)}
        ours = our_onnx.get_onnx_node(node.schema.name)(node.label, **attrs)
        for e in state.in_edges(node):
            d = sdfg.arrays[e.data.data]
            s.arrays.setdefault(e.data.data, OurArray(d.shape, _to_torch[d.dtype], strides=d.strides))
            ours.add_in_connector(e.dst_conn)
            st.add_edge(st.add_read(e.data.data), None, ours, e.dst_conn, s.make_array_memlet(e.data.data))
        for e in state.out_edges(node):
            d = sdfg.arrays[e.data.data]
            s.arrays.setdefault(e.data.data, OurArray(d.shape, _to_torch[d.dtype], strides=d.strides))
            ours.add_out_connector(e.src_conn)
            st.add_edge(ours, e.src_conn, st.add_write(e.data.data), None, s.make_array_memlet(e.data.data))
        return ours, st, s

    registered = []
    for impl, args in list(OurONNXForward.extensions().items()):
        if args.get("name") != "hip" or not donnx.has_onnx_node(args["op"]):
            continue  # fused node types (LayerNormalization, FusedEinsum ...) have no opset-12 class upstream
        op = args["op"]

        def make(op=op, impl=impl):
            class HipImplementation(RefONNXForward):
                environments = [DaceMLHip]

                @staticmethod
                def forward_can_be_applied(node, state, sdfg) -> bool:
                    try:
                        ours, st, s = mirror(node, state, sdfg)
                        return impl.forward_can_be_applied(ours, st, s)
                    except Exception:
                        return False

                @staticmethod
                def forward(node, state, sdfg):
                    ours, st, s = mirror(node, state, sdfg)
                    tasklet = impl.forward(ours, st, s)
                    ins = {c: dace.pointer(sdfg.arrays[next(state.in_edges_by_connector(node, c)).data.data].dtype)
                           for c in tasklet.in_connectors}
                    outs = {c: dace.pointer(sdfg.arrays[next(state.out_edges_by_connector(node, c)).data.data].dtype)
                            for c in tasklet.out_connectors}
                    code = render_tasklet_code(tasklet, conn_ptr=lambda c: "_" + c)
                    t = dnodes.Tasklet(node.label + "_hip", {"_" + k: v for k, v in ins.items()},
                                       {"_" + k: v for k, v in outs.items()}, code, dace.dtypes.Language.CPP)
                    t.environments = {DaceMLHip.full_class_path()}
                    return t

            HipImplementation.__name__ = "Hip" + op
            return HipImplementation

        cls = ref_op_implementation(op=op, name="hip")(make())

        class Expansion(ExpandTransformation):
            environments = [DaceMLHip]
            forward_impl = cls

            @classmethod
            def expansion(c, node, state, sdfg, **kwargs):
                node.validate(sdfg, state)
                if c.forward_impl.forward_can_be_applied(node, state, sdfg):
                    return c.forward_impl.forward(node, state, sdfg, **kwargs)
                # keep the reference's behaviour: fall back to whatever it would have used
                return type(node).implementations["onnxruntime"].expansion(node, state, sdfg, **kwargs)

        getattr(donnx, "ONNX" + op).register_implementation("hip", Expansion)
        registered.append(op)
    return registered
