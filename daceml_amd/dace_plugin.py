"""Registers the "hip" implementations inside a real DaCeML installation.

Only meaningful where ``dace`` and ``daceml`` import. Neither does in the build image, so the functions that touch
the DaCe API (``install`` and what it calls with a ``dace`` argument) have not been executed; they follow the cuDNN
expansion (daceml/onnx/op_implementations/cudnn_implementations.py:123-410), its environment
(daceml/onnx/environments/cudnn.py:11-70) and the cuDNN reverse node (daceml/autodiff/implementations/onnx_ops.py:
494-760) call by call. Everything that decides WHAT is emitted - the C++ of every tasklet, the arrays and connector
names of every nested SDFG - is computed by ``daceml_amd.lowering`` without DaCe and is covered by host-side tests
that compile the emitted code against ``include/daceml_hip.h``.

``install()``:
  1. defines a ``@dace.library.environment`` that adds ``include/`` and links ``libdaceml_hip.so``; its per-SDFG
     state holds one workspace buffer;
  2. for every "hip" implementation in this package's ``ONNXForward`` registry whose operator DaCeML has a node class
     for, builds a DaCeML ``ONNXForward`` subclass: ``forward`` mirrors the node on a stand-in SDFG, runs this
     package's expansion and returns a nested SDFG that holds one C++ tasklet with pointer connectors
     (``empty_sdfg_for_node`` + ``add_tasklet``, cudnn_implementations.py:384-410);
  3. registers it twice - ``@op_implementation`` (so autodiff's registry lookups see it) and
     ``donnx.ONNX<Op>.register_implementation`` wrapped like onnx_op.py:668-697 (node classes snapshot the registry
     at import time, so the decorator alone is not enough);
  4. registers a DaCeML ``BackwardImplementation`` (``@autoregister_params(op=..., name="hip")``,
     daceml/autodiff/base_abc.py:63-159) for every "hip" backward implementation of this package: its ``backward``
     lowers this package's reverse nodes to C++ tasklets in a nested SDFG added to the backward state, named by the
     connector contract of base_abc.py:75-108. Without this step the generator re-expands forward nodes with "pure"
     implementations and differentiates their tasklets (backward_pass_generator.py:425-494), bypassing the kernels.
After ``install()``, ``donnx.default_implementation = "hip"`` (or ``node.implementation = "hip"``) selects the
kernels for existing SDFGs, the PyTorch frontend and autodiff-generated nodes; ``node.backward_implementation =
"hip"`` (or ``ONNX<Op>.default_backward_implementation``) selects the reverse nodes.

The fused node types (LayerNormalization, Gelu, FusedEinsum, FusedAttention ...) have no opset-12 class upstream, so
they are not reached node by node. Two ways reach them a state at a time; both mirror the state's ONNX library nodes
into this package's SDFG and run its fusion pass (the role ``ReplacementTransformation``,
daceml/transformation/replacement.py:67-181, plays for single-node patterns upstream):

* ``fuse_for_training`` / ``fuse_library_nodes`` write the fused graph back as LIBRARY nodes - DaCeML's own classes
  where it has one, ``make_fused_node_class``'s generic node otherwise, whose reverse is registered for the class
  (``node_type=``, the registry form of daceml/autodiff/implementations/dace_nodes.py). Meant as a ``post_onnx_hook``
  of the reference's ``DaceModule(backward=True)``: its backward-pass generator runs after the hooks and gives every
  fused node its "hip" reverse, so training graphs run on the fused kernels in both directions.
* ``fuse_and_expand`` / ``fuse_state`` go one step further for inference modules: the fused state is expanded and
  spliced back as ONE nested SDFG of C++ tasklets (in place of ``auto_optimize``).
"""
import copy
import os

from . import lowering
from .lowering import render_tasklet_code  # noqa: F401  (public: the C++ body of one expansion)

_ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
_LIB_DIR = os.path.join(_ROOT, "daceml_amd", "csrc")

#: bytes of the per-SDFG workspace the environment allocates (every workspace query of the BERT-large and MBConv
#: configurations is far below it; a tasklet whose expansion needs more is refused at expansion time)
WORKSPACE_BYTES = 256 << 20

ENVIRONMENT_INIT_CODE = """\
__state->dmlhip_workspace_bytes = %dull;
__state->dmlhip_workspace = nullptr;
if (hipMalloc(&__state->dmlhip_workspace, __state->dmlhip_workspace_bytes) != hipSuccess)
    throw std::runtime_error("daceml_amd: cannot allocate the kernel workspace");
""" % WORKSPACE_BYTES
ENVIRONMENT_FINALIZE_CODE = "if (__state->dmlhip_workspace) (void)hipFree(__state->dmlhip_workspace);\n"
ENVIRONMENT_STATE_FIELDS = ["void* dmlhip_workspace;", "size_t dmlhip_workspace_bytes;"]
ENVIRONMENT_HEADERS = ["daceml_hip.h", "hip/hip_runtime_api.h", "stdexcept", "string"]


def _torch_dtypes(dace):
    import torch
    return {dace.float16: torch.float16, dace.float32: torch.float32, dace.float64: torch.float64,
            dace.int64: torch.int64, dace.int32: torch.int32, dace.bool: torch.bool, dace.uint8: torch.uint8}


def _dace_dtypes(dace):
    return {v: k for k, v in _torch_dtypes(dace).items()}


def make_environment(dace):
    """Links libdaceml_hip.so (pattern: daceml/onnx/environments/cudnn.py:11-49)."""
    import dace.library

    @dace.library.environment
    class DaceMLHip:
        cmake_minimum_version = None
        cmake_packages = []
        cmake_variables = {}
        cmake_includes = [os.path.join(_ROOT, "include"), "/opt/rocm/include"]
        cmake_libraries = [os.path.join(_LIB_DIR, "libdaceml_hip.so")]
        cmake_compile_flags = ["-D__HIP_PLATFORM_AMD__"]
        cmake_link_flags = ["-L" + _LIB_DIR, "-Wl,-rpath," + _LIB_DIR]
        cmake_files = []
        state_fields = list(ENVIRONMENT_STATE_FIELDS)
        headers = list(ENVIRONMENT_HEADERS)
        init_code = ENVIRONMENT_INIT_CODE
        finalize_code = ENVIRONMENT_FINALIZE_CODE
        dependencies = []

    return DaceMLHip


# ----------------------------------------------------------------------------- DaCe -> this package
def mirror_node(dace, our_onnx, node, state, sdfg):
    """Rebuild `node` with this package's classes on a one-node stand-in SDFG (descriptors only). Returns
    (our node, our state, our SDFG); arrays keep their outer names."""
    from .sdfg import SDFG as OurSDFG
    s = OurSDFG(node.label)
    st = s.add_state()
    ours = _mirror_into(dace, our_onnx, node, state, sdfg, s, st)
    return ours, st, s


def node_kind_and_attributes(our_onnx, node):
    """(operator name, attributes) of a DaCeML ONNX node or of a fused node made by ``make_fused_node_class``."""
    import json
    if hasattr(node, "hip_kind"):
        return node.hip_kind, _attributes_from_json(json.loads(node.hip_attributes or "{}"))
    cls = our_onnx.get_onnx_node(node.schema.name)
    return node.schema.name, {a: getattr(node, a) for a in cls.schema.attributes
                              if hasattr(node, a) and getattr(node, a) is not None}


def _attributes_to_json(attrs):
    """Attribute values as JSON can hold them (tuples become lists; restored by ``_attributes_from_json``)."""
    out = {}
    for k, v in attrs.items():
        if isinstance(v, tuple):
            v = {"__tuple__": [list(x) if isinstance(x, tuple) else x for x in v]}
        out[k] = v
    return out


def _attributes_from_json(attrs):
    out = {}
    for k, v in attrs.items():
        if isinstance(v, dict) and "__tuple__" in v:
            v = tuple(tuple(x) if isinstance(x, list) else x for x in v["__tuple__"])
        out[k] = v
    return out


def _mirror_into(dace, our_onnx, node, state, sdfg, s, st):
    from .sdfg import Array as OurArray
    to_torch = _torch_dtypes(dace)
    kind, attrs = node_kind_and_attributes(our_onnx, node)
    ours = our_onnx.get_onnx_node(kind)(node.label, **attrs)
    st.add_node(ours)
    for edges, is_input in ((state.in_edges(node), True), (state.out_edges(node), False)):
        for e in edges:
            name = e.data.data
            if name not in s.arrays:
                d = sdfg.arrays[name]
                s.arrays[name] = OurArray([int(x) for x in d.shape], to_torch[d.dtype], transient=bool(d.transient),
                                          strides=[int(x) for x in d.strides])
            if is_input:
                if e.dst_conn not in ours.in_connectors:
                    ours.add_in_connector(e.dst_conn)
                st.add_edge(st.add_read(name), None, ours, e.dst_conn, s.make_array_memlet(name))
            else:
                if e.src_conn not in ours.out_connectors:
                    ours.add_out_connector(e.src_conn)
                st.add_edge(ours, e.src_conn, st.add_write(name), None, s.make_array_memlet(name))
    return ours


# ----------------------------------------------------------------------------- this package -> DaCe
def emit_nested_sdfg(dace, program: lowering.TaskletProgram, descriptors, environment):
    """A ``dace.SDFG`` with one state that holds `program`'s tasklets as C++ tasklets between access nodes.
    `descriptors` maps array names to DaCe data descriptors to copy (arrays not listed are new transients in GPU
    global memory). Pattern: cudnn_implementations.py:384-410 (forward), onnx_ops.py:704-756 (reverse)."""
    to_dace = _dace_dtypes(dace)
    nsdfg = dace.SDFG(program.name + "_expansion")
    nstate = nsdfg.add_state()
    for name, d in program.arrays.items():
        if name in descriptors:
            desc = copy.deepcopy(descriptors[name])
            desc.transient = False
            nsdfg.add_datadesc(name, desc)
        else:
            nsdfg.add_array(name, list(d.shape), to_dace[d.dtype], strides=list(d.strides), transient=True,
                            storage=dace.StorageType.GPU_Global)
    last_write = {}   # array -> access node of its latest producer: orders the tasklets by data dependencies
    for spec in program.tasklets:
        ins = {"_" + c: dace.pointer(nsdfg.arrays[a].dtype) for c, a in spec.inputs.items()}
        outs = {"_" + c: dace.pointer(nsdfg.arrays[a].dtype) for c, a in spec.outputs.items()}
        tasklet = nstate.add_tasklet(spec.label, ins, outs, spec.code(), dace.dtypes.Language.CPP)
        tasklet.environments = {environment.full_class_path()}
        for conn, arr in spec.inputs.items():
            src = last_write.get(arr) or nstate.add_read(arr)
            nstate.add_edge(src, None, tasklet, "_" + conn, nsdfg.make_array_memlet(arr))
        for conn, arr in spec.outputs.items():
            dst = nstate.add_write(arr)
            nstate.add_edge(tasklet, "_" + conn, dst, None, nsdfg.make_array_memlet(arr))
            last_write[arr] = dst
    return nsdfg


def _check_workspace(program: lowering.TaskletProgram):
    if program.workspace_bytes > WORKSPACE_BYTES:
        raise ValueError("%s needs a workspace of %d bytes, the environment provides %d" %
                         (program.name, program.workspace_bytes, WORKSPACE_BYTES))


def forward_program(tasklet) -> lowering.TaskletProgram:
    """The TaskletProgram of one forward expansion: arrays are named after the node's connectors, as
    ``empty_sdfg_for_node`` names them (op_implementations/utils.py:105-139)."""
    if not tasklet.calls:
        raise ValueError("%r moves no data (a view): there is nothing to emit" % tasklet)
    spec = lowering.TaskletSpec(tasklet.label, {c: c for c in tasklet.in_connectors},
                                {c: c for c in tasklet.out_connectors}, list(tasklet.calls), {})
    return lowering.TaskletProgram(tasklet.label, {}, {}, [spec], int(tasklet.workspace_bytes))


# ----------------------------------------------------------------------------- installation
def install():
    """Register everything with an importable DaCeML. Raises ImportError where dace / daceml are absent. Returns
    ``{"forward": [ops], "backward": [ops]}``."""
    import dace
    from dace.transformation.transformation import ExpandTransformation
    import daceml.onnx as donnx
    from daceml.onnx.forward_implementation_abc import ONNXForward as RefONNXForward
    from daceml.onnx.op_implementations.utils import op_implementation as ref_op_implementation
    from daceml.util.utils import in_desc_with_name, out_desc_with_name

    from . import onnx as our_onnx
    from .onnx.forward_implementation_abc import ONNXForward as OurONNXForward

    env = make_environment(dace)
    registered = {"forward": [], "backward": []}
    for impl, args in list(OurONNXForward.extensions().items()):
        if args.get("name") != "hip" or not donnx.has_onnx_node(args["op"]):
            continue   # fused node types have no opset-12 class upstream: see fuse_state
        op = args["op"]

        def make(op=op, impl=impl):
            class HipImplementation(RefONNXForward):
                environments = [env]

                @staticmethod
                def forward_can_be_applied(node, state, sdfg) -> bool:
                    try:
                        ours, st, s = mirror_node(dace, our_onnx, node, state, sdfg)
                        if not impl.forward_can_be_applied(ours, st, s):
                            return False
                        _check_workspace(forward_program(impl.forward(ours, st, s)))
                        return True
                    except Exception:
                        return False

                @staticmethod
                def forward(node, state, sdfg):
                    ours, st, s = mirror_node(dace, our_onnx, node, state, sdfg)
                    program = forward_program(impl.forward(ours, st, s))
                    _check_workspace(program)
                    descs = {}
                    for e in state.in_edges(node):
                        descs[e.dst_conn] = in_desc_with_name(node, state, sdfg, e.dst_conn)
                    for e in state.out_edges(node):
                        descs[e.src_conn] = out_desc_with_name(node, state, sdfg, e.src_conn)
                    from .sdfg import Array as OurArray
                    to_torch = _torch_dtypes(dace)
                    program.arrays = {c: OurArray([int(x) for x in d.shape], to_torch[d.dtype]) for c, d in descs.items()}
                    return emit_nested_sdfg(dace, program, descs, env)

            HipImplementation.__name__ = "Hip" + op
            return HipImplementation

        cls = ref_op_implementation(op=op, name="hip")(make())

        def make_expansion(cls=cls):
            class Expansion(ExpandTransformation):
                environments = [env]
                forward_impl = cls

                @classmethod
                def expansion(c, node, state, sdfg, **kwargs):
                    node.validate(sdfg, state)
                    if c.forward_impl.forward_can_be_applied(node, state, sdfg):
                        return c.forward_impl.forward(node, state, sdfg, **kwargs)
                    # keep the reference's behaviour: fall back to what it would have used (onnx_op.py:685-697)
                    return type(node).implementations["onnxruntime"].expansion(node, state, sdfg, **kwargs)

            return Expansion

        getattr(donnx, "ONNX" + op).register_implementation("hip", make_expansion())
        registered["forward"].append(op)

    registered["backward"] = _install_backward(dace, donnx, our_onnx, env)
    return registered


def _backward_tools(dace, our_onnx, env):
    """(lowered, emit): the two halves every reverse-node registration shares. `lowered` runs one of this package's
    backward implementations on a mirror of the forward node and lowers what it adds; `emit` turns the result into a
    nested SDFG in the backward state (pattern: the cuDNN reverse node, onnx_ops.py:704-756)."""
    from daceml.autodiff.base_abc import BackwardResult as RefBackwardResult
    import daceml.autodiff.utils as butils

    def lowered(impl, forward_node, state, sdfg, given, required):
        ours, st, s = mirror_node(dace, our_onnx, forward_node, state, sdfg)
        if not impl.backward_can_be_applied(ours, st, s):
            raise ValueError("not applicable")
        lb = lowering.lower_backward(ours, st, s, impl, given, required)
        _check_workspace(lb.program)
        return lb

    def emit(impl, forward_node, context, given_gradients, required_gradients):
        lb = lowered(impl, forward_node, context.forward_state, context.forward_sdfg, list(given_gradients),
                     list(required_gradients))
        descs = {}
        for conn in lb.forward_inputs:
            descs[conn] = butils.forward_in_desc_with_name(forward_node, context, conn)
        for conn in lb.forward_outputs:
            descs[conn] = butils.forward_out_desc_with_name(forward_node, context, conn)
        for conn, name in lb.given_grad_names.items():
            descs[name] = butils.forward_out_desc_with_name(forward_node, context, conn)
        for conn, name in lb.required_grad_names.items():
            descs[name] = butils.forward_in_desc_with_name(forward_node, context, conn)
        nsdfg = emit_nested_sdfg(dace, lb.program, descs, env)
        inputs = set(lb.forward_inputs) | set(lb.forward_outputs) | set(lb.given_grad_names.values())
        outputs = set(lb.required_grad_names.values())
        node = context.backward_state.add_nested_sdfg(nsdfg, None, inputs, outputs)
        # forward inputs are connected by the generator (connectors named like the forward node's);
        # forward outputs have to be asked for (autodiff/utils.py:224-261)
        for conn in lb.forward_outputs:
            butils.connect_output_from_forward(forward_node, node, context, conn)
        # every gradient is written in full by its kernel: nothing has to be zeroed first
        zero_init = {name: False for name in lb.required_grad_names.values()}
        return node, RefBackwardResult(required_grad_names=dict(lb.required_grad_names),
                                       given_grad_names=dict(lb.given_grad_names), zero_init=zero_init)

    def applicable(impl, node, state, sdfg):
        try:
            given = [e.src_conn for e in state.out_edges(node)]
            required = [e.dst_conn for e in state.in_edges(node)
                        if sdfg.arrays[e.data.data].dtype in (dace.float16, dace.float32)]
            lowered(impl, node, state, sdfg, given, required)
            return True
        except Exception:
            if os.environ.get("DACEML_AMD_DEBUG"):
                import traceback
                traceback.print_exc()
            return False

    return applicable, emit


def _hip_backward_implementations():
    """{operator name: this package's "hip" backward implementation}."""
    from .autodiff.base_abc import BackwardImplementation as OurBackwardImplementation
    return {args["op"]: impl for impl, args in OurBackwardImplementation.extensions().items()
            if args.get("name") == "hip" and args.get("op") is not None}


def _install_backward(dace, donnx, our_onnx, env):
    import dace.registry
    from daceml.autodiff.base_abc import BackwardImplementation as RefBackwardImplementation

    applicable, emit = _backward_tools(dace, our_onnx, env)
    done = []
    for op, impl in _hip_backward_implementations().items():
        if not donnx.has_onnx_node(op):
            continue

        def make(op=op, impl=impl):
            class HipBackward(RefBackwardImplementation):
                @staticmethod
                def backward_can_be_applied(node, state, sdfg) -> bool:
                    return applicable(impl, node, state, sdfg)

                @staticmethod
                def backward(forward_node, context, given_gradients, required_gradients):
                    return emit(impl, forward_node, context, given_gradients, required_gradients)

            HipBackward.__name__ = "Hip%sBackward" % op
            return HipBackward

        dace.registry.autoregister_params(op=op, name="hip")(make())
        done.append(op)
    return done


# ----------------------------------------------------------------------------- fused nodes as library nodes
_FUSED_NODE_CLASS = {}


def make_fused_node_class(dace, env=None):
    """ONE DaCe library node class for every node type the fusion pass creates that DaCeML has no opset-12 class for
    (LayerNormalization, Gelu, BiasGelu, FusedEinsum, FusedAttention, ...): ``hip_kind`` names the type,
    ``hip_attributes`` holds its attributes as JSON (both are DaCe properties, so the node survives SDFG
    serialisation). Its only expansion mirrors the node into this package and emits the nested SDFG of C++ tasklets,
    exactly as the per-operator "hip" implementations do; its reverse is registered for the CLASS
    (``@autoregister_params(node_type=HipFusedNode, name="hip")``: the registry form DaCeML uses for DaCe's own
    library nodes, daceml/autodiff/implementations/dace_nodes.py:13-19, looked up by
    ``find_backward_implementation``, daceml/autodiff/base_abc.py:114-159) and dispatches on ``hip_kind``.

    A graph that holds these nodes is still a graph of library nodes: the reference's backward-pass generator, which
    runs AFTER the post-ONNX hooks, finds a reverse for each of them instead of expanding and differentiating
    tasklets (backward_pass_generator.py:425-494). That is what makes the fused kernels reachable from modules built
    with ``backward=True``."""
    if dace in _FUSED_NODE_CLASS:
        return _FUSED_NODE_CLASS[dace]
    import json
    import dace.library
    import dace.registry
    from dace.properties import Property
    from dace.transformation.transformation import ExpandTransformation
    from daceml.autodiff.base_abc import BackwardImplementation as RefBackwardImplementation
    from daceml.util.utils import in_desc_with_name, out_desc_with_name

    from . import onnx as our_onnx
    from .onnx.forward_implementation_abc import ONNXForward as OurONNXForward
    from .sdfg import Array as OurArray
    env = env or make_environment(dace)
    forward_impls = {args["op"]: impl for impl, args in OurONNXForward.extensions().items() if args.get("name") == "hip"}

    @dace.library.expansion
    class ExpandHip(ExpandTransformation):
        environments = [env]

        @staticmethod
        def expansion(node, state, sdfg, **kwargs):
            impl = forward_impls[node.hip_kind]
            ours, st, s = mirror_node(dace, our_onnx, node, state, sdfg)
            if not impl.forward_can_be_applied(ours, st, s):
                raise ValueError("%s (%s): the HIP implementation does not apply to these operands" %
                                 (node.label, node.hip_kind))
            program = forward_program(impl.forward(ours, st, s))
            _check_workspace(program)
            descs = {e.dst_conn: in_desc_with_name(node, state, sdfg, e.dst_conn) for e in state.in_edges(node)}
            descs.update({e.src_conn: out_desc_with_name(node, state, sdfg, e.src_conn) for e in state.out_edges(node)})
            to_torch = _torch_dtypes(dace)
            program.arrays = {c: OurArray([int(x) for x in d.shape], to_torch[d.dtype]) for c, d in descs.items()}
            return emit_nested_sdfg(dace, program, descs, env)

    @dace.library.node
    class HipFusedNode(dace.nodes.LibraryNode):
        implementations = {"hip": ExpandHip}
        default_implementation = "hip"
        hip_kind = Property(dtype=str, default="", desc="node type of daceml_amd (LayerNormalization, Gelu, ...)")
        hip_attributes = Property(dtype=str, default="{}", desc="the node's attributes, JSON")

        def __init__(self, name, kind="", attributes=None, inputs=(), outputs=(), **kwargs):
            super().__init__(name, inputs=set(inputs), outputs=set(outputs), **kwargs)
            self.hip_kind = kind
            self.hip_attributes = json.dumps(_attributes_to_json(attributes or {}), sort_keys=True)

    applicable, emit = _backward_tools(dace, our_onnx, env)
    backward_impls = _hip_backward_implementations()

    class HipFusedBackward(RefBackwardImplementation):
        @staticmethod
        def backward_can_be_applied(node, state, sdfg) -> bool:
            impl = backward_impls.get(node.hip_kind)
            return impl is not None and applicable(impl, node, state, sdfg)

        @staticmethod
        def backward(forward_node, context, given_gradients, required_gradients):
            return emit(backward_impls[forward_node.hip_kind], forward_node, context, given_gradients,
                        required_gradients)

    dace.registry.autoregister_params(node_type=HipFusedNode, name="hip")(HipFusedBackward)
    _FUSED_NODE_CLASS[dace] = HipFusedNode
    return HipFusedNode


def _forward_outputs_the_reverse_needs(node, st, s):
    """[(connector, shape, dtype)] of optional outputs (statistics, log-sum-exp, pre-activation) that the "hip" reverse
    of `node` asks its forward node for and `node` does not have yet: found by running the reverse on a copy."""
    import copy
    from .autodiff.base_abc import BackwardContext
    impl = _hip_backward_implementations().get(node.schema.name)
    if impl is None:
        return []
    s2 = copy.deepcopy(s)
    st2 = next(x for x in s2.states() if x.label == st.label)
    node2 = next(n for n in st2.library_nodes() if n.label == node.label)
    try:
        if not impl.backward_can_be_applied(node2, st2, s2):
            return []
        given = [e.src_conn for e in st2.out_edges(node2)]
        required = [e.dst_conn for e in st2.in_edges(node2) if s2.arrays[e.data.data].dtype.is_floating_point]
        before = set(node2.out_connectors)
        impl.backward(node2, BackwardContext(s2, st2, s2, s2.add_state(node.label + "_probe"), None), given, required)
    except Exception:
        return []
    extra = []
    for e in st2.out_edges(node2):
        if e.src_conn not in before:
            d = s2.arrays[e.data.data]
            extra.append((e.src_conn, tuple(d.shape), d.dtype))
    return extra


def fuse_library_nodes(sdfg, state, training: bool = True, environment=None, constants=None):
    """Rewrite `state` (ONNX library nodes and access nodes only) into its fused form WITHOUT leaving the level of
    library nodes: the state is mirrored, run through this package's fusion pass, and written back - node types
    DaCeML has a class for as ``donnx.ONNX<Op>`` nodes, the others as nodes of ``make_fused_node_class``. With
    `training` the fused nodes are created with the optional outputs their reverse nodes read (LayerNormalization's
    Mean / InvStdDev, FusedAttention's LogSumExp, the pre-activation of a contraction with a folded Gelu), because a
    reverse node registered with DaCeML can ask for outputs the forward node has (``connect_output_from_forward``)
    but cannot add any. Transposes next to contractions are folded into their equations; Reshape nodes stay nodes (they
    are not turned into strided views: DaCe has its own view mechanism). `constants`: see ``mirror_state``. The counterpart of
    ``ReplacementTransformation`` (daceml/transformation/replacement.py:67-181) for whole states. Returns how often
    each rewrite fired."""
    import dace
    import daceml.onnx as donnx
    from . import onnx as our_onnx
    from .sdfg import AccessNode as OurAccessNode
    from .transformation import fusion
    env = environment or make_environment(dace)
    fused_cls = make_fused_node_class(dace, env)
    to_dace = _dace_dtypes(dace)
    st, s = mirror_state(dace, our_onnx, state, sdfg, constants)
    stats = fusion.auto_optimize(s, training=training, views=False)
    if training:
        for node in list(st.library_nodes()):
            for conn, shape, dtype in _forward_outputs_the_reverse_needs(node, st, s):
                name, _ = s.add_transient("%s_%s" % (node.label, conn), shape, dtype)
                node.add_out_connector(conn)
                st.add_edge(node, conn, st.add_write(name), None, s.make_array_memlet(name))
    for name, d in s.arrays.items():
        if name not in sdfg.arrays:
            sdfg.add_array(name, list(d.shape), to_dace[d.dtype], strides=list(d.strides), transient=True,
                           storage=dace.StorageType.GPU_Global, find_new_name=False)
    for node in list(state.nodes()):
        state.remove_node(node)
    last_write = {}
    for node in st.topological_sort():
        if isinstance(node, OurAccessNode):
            continue
        kind = node.schema.name
        attrs = {a: getattr(node, a) for a in node.schema.attributes if getattr(node, a, None) is not None}
        ins = {e.dst_conn: e.data.data for e in st.in_edges(node)}
        outs = {e.src_conn: e.data.data for e in st.out_edges(node)}
        if donnx.has_onnx_node(kind):
            new = getattr(donnx, "ONNX" + kind)(node.label, **attrs)
            for conn in list(ins) + list(outs):   # variadic connectors are added on demand upstream as well
                pool, add = (new.in_connectors, new.add_in_connector) if conn in ins else (new.out_connectors,
                                                                                          new.add_out_connector)
                if conn not in pool:
                    add(conn)
        else:
            new = fused_cls(node.label, kind=kind, attributes=attrs, inputs=ins, outputs=outs)
        state.add_node(new)
        for conn, arr in ins.items():
            src = last_write.get(arr) or state.add_read(arr)
            state.add_edge(src, None, new, conn, sdfg.make_array_memlet(arr))
        for conn, arr in outs.items():
            dst = state.add_write(arr)
            state.add_edge(new, conn, dst, None, sdfg.make_array_memlet(arr))
            last_write[arr] = dst
    return stats


def fuse_for_training(dace_module):
    """``post_onnx_hook`` for the reference's ``DaceModule(..., backward=True)`` (daceml/torch/module.py:179-245; the
    hooks run before the backward pass is generated, :333-346): every state of ONNX library nodes is rewritten by
    ``fuse_library_nodes``. With ``install()`` done and ``donnx.default_implementation = "hip"``, forward runs on the
    fused kernels and the generator gives every fused node its "hip" reverse."""
    from .onnx.onnx_importer import clean_onnx_name
    sdfg = dace_module.sdfg
    weights = getattr(getattr(dace_module, "dace_model", None), "weights", None) or {}
    constants = {clean_onnx_name(n): t for n, t in weights.items()}
    fused = 0
    for state in sdfg.nodes():
        try:
            fuse_library_nodes(sdfg, state, training=True, constants=constants)
            fused += 1
        except ValueError:
            continue
    return fused


# ----------------------------------------------------------------------------- fused states
def mirror_state(dace, our_onnx, state, sdfg, constants=None):
    """All ONNX library nodes of `state` on a stand-in SDFG of this package. Raises ``ValueError`` if the state
    holds anything other than ONNX library nodes this package has classes for and access nodes. `constants`: values
    of arrays that are compile-time constants ({array name: tensor}; the importer of the reference keeps them in
    ``ONNXModel.weights``, onnx_importer.py:340-388); single-element ones are made known to the fusion pass, which
    reads the epsilon of a LayerNorm chain, the exponent of its Pow, the sqrt(2) of a Gelu chain from them."""
    from daceml.onnx.nodes.onnx_op import ONNXOp as RefONNXOp
    from .sdfg import SDFG as OurSDFG
    s = OurSDFG(sdfg.name + "_" + state.label)
    st = s.add_state(state.label)
    for node in state.nodes():
        if isinstance(node, dace.nodes.AccessNode):
            continue
        fused = hasattr(node, "hip_kind")
        if not fused and (not isinstance(node, RefONNXOp) or not our_onnx.has_onnx_node(node.schema.name)):
            raise ValueError("state %s holds %r, which has no counterpart here" % (state.label, node))
        _mirror_into(dace, our_onnx, node, state, sdfg, s, st)
    for name, value in (constants or {}).items():
        if name in s.arrays and hasattr(value, "numel") and value.numel() == 1 and not s.arrays[name].transient:
            s.add_constant(name, value.detach().reshape(s.arrays[name].shape).to(s.arrays[name].dtype))
    return st, s


def fuse_state(sdfg, state, training: bool = False, environment=None):
    """Replace the contents of `state` (ONNX library nodes and access nodes only) by one nested SDFG of C++ tasklets:
    the state is mirrored, fused (``transformation.fusion.auto_optimize``), expanded with the "hip" implementations
    and lowered. Returns the nested SDFG node. Arrays that the fused state no longer touches stay in `sdfg`."""
    import dace
    from . import onnx as our_onnx
    from .runtime import expand_onnx_nodes
    from .transformation import fusion
    env = environment or make_environment(dace)
    st, s = mirror_state(dace, our_onnx, state, sdfg)
    # arrays that other states or the caller see must survive fusion as they are
    fusion.auto_optimize(s, training=training)
    expand_onnx_nodes(s)
    program = lowering.lower_state(s, st, name=sdfg.name + "_" + state.label + "_fused")
    _check_workspace(program)
    descs = {n: sdfg.arrays[n] for n in program.arguments() if n in sdfg.arrays}
    missing = [n for n in program.arguments() if n not in descs]
    if missing:
        raise ValueError("the fused state reads arrays the SDFG does not have: %s" % missing)
    nsdfg = emit_nested_sdfg(dace, program, descs, env)
    reads = {a for t in program.tasklets for a in t.inputs.values() if a in descs}
    writes = {a for t in program.tasklets for a in t.outputs.values() if a in descs}
    for node in list(state.nodes()):
        state.remove_node(node)
    nested = state.add_nested_sdfg(nsdfg, sdfg, reads, writes)
    for name in sorted(reads):
        state.add_edge(state.add_read(name), None, nested, name, sdfg.make_array_memlet(name))
    for name in sorted(writes):
        state.add_edge(nested, name, state.add_write(name), None, sdfg.make_array_memlet(name))
    return nested


def fuse_and_expand(dace_module):
    """``post_onnx_hook`` for the reference's ``DaceModule`` (daceml/torch/module.py:179-245) in place of
    ``auto_optimize``: every state that consists of ONNX library nodes is replaced by its fused form; states that hold
    anything else are left to the node-by-node expansions. Inference modules only: the reference differentiates AFTER
    its post-ONNX hooks, and a state of C++ tasklets cannot be differentiated - modules built with ``backward=True``
    use ``fuse_for_training``, which stays at the level of library nodes."""
    if getattr(dace_module, "backward", False):
        raise ValueError("fuse_and_expand is for inference modules; with backward=True use fuse_for_training "
                         "(fused library nodes with registered reverse nodes) after install()")
    sdfg = dace_module.sdfg
    fused = 0
    for state in sdfg.nodes():
        try:
            fuse_state(sdfg, state)
            fused += 1
        except ValueError:
            continue
    return fused
