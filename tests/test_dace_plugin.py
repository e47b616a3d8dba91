"""The path into a real DaCeML, as far as it can be checked without DaCe: every expansion and every reverse node is
lowered to the C++ its tasklets would hold, and that code is compiled against include/daceml_hip.h with the host
compiler (signature drift between the Python-side call specifications and the C ABI shows up as a compile error);
the registration logic of ``dace_plugin.install`` runs against small recording stand-ins of the ``dace`` / ``daceml``
modules, which checks its control flow and naming, not the fidelity of the stand-ins to DaCe."""
import copy
import os
import subprocess
import sys
import types

import numpy as np
import pytest
import torch

from daceml_amd import graphs, lowering
from daceml_amd.autodiff import add_backward_pass
from daceml_amd.autodiff.base_abc import BackwardImplementation, find_backward_implementation
from daceml_amd.onnx.forward_implementation_abc import ONNXForward
from daceml_amd.onnx.nodes import NotApplicable, ONNXOp
from daceml_amd.runtime import expand_onnx_nodes
from daceml_amd.transformation import fusion

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
INCLUDE = os.path.join(ROOT, "include")
LIBDIR = os.path.join(ROOT, "daceml_amd", "csrc")


# ----------------------------------------------------------------------------- sample graphs
def _unary_graph(dtype, differentiable=False):
    """A chain through the unary maps, the reductions and the odd ones out; `differentiable` leaves out the operators
    that have no reverse node (ReduceMax / ReduceMin / Identity / Sum / Cast)."""
    g = graphs.GraphBuilder("unary", dtype)
    x = g.input("x", (4, 64))
    cur = x
    for op, i, o in (("Erf", "input", "output"), ("Sqrt", "X", "Y"), ("Exp", "input", "output"),
                     ("Log", "input", "output"), ("Tanh", "input", "output"), ("Relu", "X", "Y"),
                     ("Sigmoid", "X", "Y"), ("Reciprocal", "X", "Y"), ("Identity", "input", "output")):
        if differentiable and op == "Identity":
            continue
        cur = g.node(op, {i: cur}, {o: (4, 64)}, label=op.lower())[o]
    for op in (("ReduceSum", "ReduceMean") if differentiable else ("ReduceMax", "ReduceMin", "ReduceSum", "ReduceMean")):
        r = g.node(op, {"data": cur}, {"reduced": (4, 1)}, label=op.lower(), axes=[1], keepdims=1)["reduced"]
        cur = g.node("Sub", {"A": cur, "B": r}, {"C": (4, 64)}, label=op.lower() + "_sub")["C"]
    two = g.constant("two", 2.0)
    cur = g.node("Pow", {"X": cur, "Y": two}, {"Z": (4, 64)}, label="pow")["Z"]
    cur = g.node("Div", {"A": cur, "B": x}, {"C": (4, 64)}, label="div")["C"]
    if differentiable:
        g.output(cur, "y")
        return g.sdfg
    s = g.node("Sum", {"data_0__0": cur, "data_0__1": x}, {"sum": (4, 64)}, label="sum")["sum"]
    c = g.node("Cast", {"input": s}, {"output": (4, 64)}, label="cast", out_dtype=torch.float32 if dtype == torch.float16
               else torch.float16, to=1 if dtype == torch.float16 else 10)["output"]
    g.output(c, "y")
    return g.sdfg


def _gemm_graph(dtype, beta, c_shape):
    g = graphs.GraphBuilder("gemm", dtype)
    a, b = g.input("a", (64, 24)), g.input("b", (64, 40))
    ins = {"A": a, "B": b}
    if c_shape is not None:
        ins["C"] = g.input("c", c_shape)
    y = g.node("Gemm", ins, {"Y": (24, 40)}, label="gemm", alpha=0.5, beta=beta, transA=1, transB=0)["Y"]
    g.output(y, "y")
    return g.sdfg


def _batchnorm_graph():
    g = graphs.GraphBuilder("bn", torch.float32)
    x = g.input("x", (4, 6, 8, 8))
    for name in ("scale", "bias", "mean", "var"):
        g.input(name, (6, ))
    outs = g.node("BatchNormalization", {"X": x, "scale": "scale", "B": "bias", "in_mean": "mean", "in_var": "var"},
                  {"Y": (4, 6, 8, 8), "out_mean": (6, ), "out_var": (6, ), "saved_mean": (6, ), "saved_var": (6, )},
                  label="bn", epsilon=1e-5, momentum=0.9)
    g.output(g.swish(outs["Y"], "act"), "y")
    return g


def _sample_sdfgs():
    """(name, SDFG with unexpanded library nodes) pairs that between them use every "hip" implementation."""
    out = []
    for dtype, tag in ((torch.float16, "f16"), (torch.float32, "f32")):
        out.append(("bert_unfused_" + tag, graphs.bert_encoder_layer(2, 64, 256, 4, 512, dtype)))
        for attention in (True, False):
            s = graphs.bert_encoder_layer(2, 64, 256, 4, 512, dtype)
            fusion.auto_optimize(s, training=True, attention=attention, gelu_epilogue=not attention)
            add_backward_pass(s, s.states()[0], ["y"], ["x"] + graphs.BERT_PARAM_NAMES,
                              grad_dtypes={n: torch.float32 for n in graphs.BERT_PARAM_NAMES})
            if attention:
                fusion.optimize_backward(s)
            out.append(("bert_train_%s_attention%d" % (tag, attention), s))
        s = graphs.bert_encoder_layer(2, 64, 256, 4, 512, dtype)
        fusion.auto_optimize(s)
        out.append(("bert_inference_" + tag, s))
        out.append(("unary_" + tag, _unary_graph(dtype)))
        s = _unary_graph(dtype, differentiable=True)
        add_backward_pass(s, s.states()[0], ["y"], ["x"])
        out.append(("unary_backward_" + tag, s))
        for beta, c_shape in ((0.0, None), (1.0, (40, )), (1.0, (24, 40)), (0.5, (40, )), (0.5, (24, 40)), (2.0, (1, 40))):
            out.append(("gemm_%s_beta%g_%s" % (tag, beta, c_shape), _gemm_graph(dtype, beta, c_shape)))
    s = graphs.mbconv_block(2, 16, 32, expand=6, cout=24, se_reduce=4, stride=2, dtype=torch.float32)
    out.append(("mbconv_unfused", copy.deepcopy(s)))
    t = copy.deepcopy(s)
    fusion.auto_optimize(t)
    out.append(("mbconv_inference", t))
    t = copy.deepcopy(s)
    fusion.auto_optimize(t, training=True)
    params = [n for n in t.arglist() if n not in ("y", )]
    add_backward_pass(t, t.states()[0], ["y"], params)
    fusion.optimize_backward(t)
    out.append(("mbconv_train", t))
    g = _batchnorm_graph()
    fusion.auto_optimize(g.sdfg, training=True)
    add_backward_pass(g.sdfg, g.state, ["y"], ["x", "scale", "bias"])
    out.append(("batchnorm_train", g.sdfg))
    g = _batchnorm_graph()
    out.append(("batchnorm_unfused", g.sdfg))
    g = graphs.GraphBuilder("bias_gelu", torch.float16)
    x = g.input("x", (4, 8, 64))
    g.input("b", (64, ))
    h = g.node("Add", {"A": "b", "B": x}, {"C": (4, 8, 64)}, label="bias")["C"]
    g.output(g.gelu(h, "gelu"), "y")
    fusion.auto_optimize(g.sdfg)
    out.append(("bias_gelu_chain", g.sdfg))
    # the two fused node types that are only built directly / from a residual Add no contraction absorbed
    g = graphs.GraphBuilder("bias_gelu_node", torch.float16)
    x = g.input("x", (4, 8, 64))
    g.input("b", (64, ))
    g.output(g.node("BiasGelu", {"A": x, "B": "b"}, {"C": (4, 8, 64)}, label="bg")["C"], "y")
    out.append(("bias_gelu_node", g.sdfg))
    g = graphs.GraphBuilder("skip_ln", torch.float16)
    x, r = g.input("x", (4, 8, 64)), g.input("r", (4, 8, 64))
    g.input("gamma", (64, ))
    g.input("beta", (64, ))
    h = g.node("Add", {"A": x, "B": r}, {"C": (4, 8, 64)}, label="res")["C"]
    g.output(g.layer_norm(h, "gamma", "beta", 1e-5, "ln"), "y")
    assert fusion.auto_optimize(g.sdfg)["skip_layernorm"] == 1
    out.append(("skip_layernorm", g.sdfg))
    # attention with an additive mask, forward and reverse
    from tests.test_zx_attention_mask import _chain
    g = _chain((2, 1, 1, 48))
    assert fusion.auto_optimize(g.sdfg)["attention"] == 1
    add_backward_pass(g.sdfg, g.state, ["o"], ["q", "k", "v"])
    out.append(("masked_attention_train", g.sdfg))
    # a Pad that does not fold into the Conv behind it (one-sided), forward and reverse
    g = graphs.GraphBuilder("pad_conv_train", torch.float32)
    p = g.node("Pad", {"data": g.input("x", (2, 3, 6, 6))}, {"output": (2, 3, 7, 8)}, label="pad",
               pads=[0, 0, 0, 2, 0, 0, 1, 0])["output"]
    g.output(g.node("Conv", {"X": p, "W": g.input("w", (4, 3, 3, 3))}, {"Y": (2, 4, 5, 6)}, label="conv",
                    kernel_shape=[3, 3])["Y"], "y")
    assert fusion.auto_optimize(g.sdfg, training=True)["pad_into_conv"] == 0
    add_backward_pass(g.sdfg, g.state, ["y"], ["x", "w"])
    out.append(("pad_conv_train", g.sdfg))
    for dtype, tag in ((torch.float16, "f16"), (torch.float32, "f32")):
        g = graphs.GraphBuilder("log_softmax_" + tag, dtype)
        g.output(g.node("LogSoftmax", {"input": g.input("x", (6, 4, 10))}, {"output": (6, 4, 10)}, label="lsm", axis=1)["output"],
                 "y")
        add_backward_pass(g.sdfg, g.state, ["y"], ["x"])
        out.append(("log_softmax_train_" + tag, g.sdfg))
        g = graphs.GraphBuilder("maxpool_" + tag, dtype)
        g.output(g.node("MaxPool", {"X": g.input("x", (2, 3, 9, 8))}, {"Y": (2, 3, 4, 3)}, label="pool", kernel_shape=[3, 3],
                        strides=[2, 2])["Y"], "y")
        add_backward_pass(g.sdfg, g.state, ["y"], ["x"])
        out.append(("maxpool_train_" + tag, g.sdfg))
    return out


# ----------------------------------------------------------------------------- compile helpers
TASKLET_HARNESS = """#include <stddef.h>
#include <stdint.h>
#include <math.h>
#include <stdexcept>
#include <string>
#include "daceml_hip.h"
struct half { uint16_t bits; };
struct __dml_state_t { void* dmlhip_workspace; size_t dmlhip_workspace_bytes; };
typedef void* hipStream_t;
"""


def _tasklet_function(index, spec, program):
    """One tasklet's code the way DaCe would host it: typed pointer connectors, the per-SDFG state struct and the
    current stream in scope."""
    params = ["__dml_state_t* __state", "hipStream_t __dace_current_stream"]
    for conn, arr in list(spec.inputs.items()) + list(spec.outputs.items()):
        params.append("%s* _%s" % (lowering.CXX_TYPES[program.arrays[arr].dtype], conn))
    return "void tasklet_%d(%s) {\n%s\n}\n" % (index, ", ".join(params), spec.code())


def _compile(source, tmp_path, name, link=False):
    path = tmp_path / (name + ".cpp")
    path.write_text(source)
    cmd = ["g++", "-std=c++17", "-Wall", "-Wno-unused-variable", "-Werror=return-type", "-I", INCLUDE]
    if link:
        cmd += ["-shared", "-fPIC", "-o", str(tmp_path / (name + ".so")), str(path), "-L", LIBDIR, "-ldaceml_hip",
                "-Wl,--no-undefined", "-Wl,-rpath," + LIBDIR]
    else:
        cmd += ["-fsyntax-only", str(path)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    assert res.returncode == 0, "%s does not compile:\n%s" % (path, res.stderr[:6000])


# ----------------------------------------------------------------------------- tests
def test_every_expansion_renders_to_code_that_compiles_against_the_header(tmp_path):
    covered, functions, n = set(), [TASKLET_HARNESS], 0
    programs = []
    for name, sdfg in _sample_sdfgs():
        for st in sdfg.states():
            covered |= {nd.schema.name for nd in st.library_nodes() if isinstance(nd, ONNXOp)}
        expand_onnx_nodes(sdfg)
        for st in sdfg.states():
            program = lowering.lower_state(sdfg, st, name="%s_%s" % (name, st.label))
            programs.append(program)
            for spec in program.tasklets:
                functions.append(_tasklet_function(n, spec, program))
                n += 1
    registered = {a["op"] for _, a in ONNXForward.extensions().items() if a.get("name") == "hip"}
    # Reshape expands to a view (no call to render)
    assert registered - covered == set(), "implementations that no sample graph uses: %s" % sorted(registered - covered)
    assert n > 150
    _compile("".join(functions), tmp_path, "tasklets")
    # the same programs as freestanding functions, compiled AND linked against the built library: every symbol a
    # rendered call names exists, with the declared signature
    source = lowering.CXX_PRELUDE + "".join(
        lowering.emit_cxx(p, function="program_%d" % i, prelude=False) for i, p in enumerate(programs))
    _compile(source, tmp_path, "programs", link=True)


def test_reverse_nodes_lower_to_stand_alone_programs(tmp_path):
    """What the plugin registers as BackwardImplementations: for every node of the un-fused BERT layer and MBConv
    block (the operators DaCeML has node classes for) the reverse is lowered on its own, with forward arrays named
    after the forward connectors and gradients after the BackwardResult connectors, and its code compiles."""
    functions, n, ops = [TASKLET_HARNESS], 0, set()
    samples = [graphs.bert_encoder_layer(2, 64, 256, 4, 512, torch.float16),
               graphs.mbconv_block(2, 16, 32, expand=6, cout=24, se_reduce=4, stride=2, dtype=torch.float32),
               _unary_graph(torch.float32, differentiable=True)]
    fusion.lower_matmul(samples[0])
    for base in samples:
        count = len([x for x in base.states()[0].topological_sort() if isinstance(x, ONNXOp)])
        for i in range(count):
            sdfg = copy.deepcopy(base)
            st = sdfg.states()[0]
            node = [x for x in st.topological_sort() if isinstance(x, ONNXOp)][i]
            impl = find_backward_implementation(sdfg, st, node)
            if impl is None:
                assert node.schema.name == "Reshape", node
                continue
            given = [e.src_conn for e in st.out_edges(node)]
            required = [e.dst_conn for e in st.in_edges(node)
                        if e.data.data not in sdfg.constants and sdfg.arrays[e.data.data].dtype.is_floating_point]
            lb = lowering.lower_backward(node, st, sdfg, impl, given, required)
            ops.add(node.schema.name)
            prog = lb.program
            assert set(lb.required_grad_names) == set(required)
            assert set(lb.given_grad_names) <= set(given) and lb.given_grad_names
            # inputs of the program: forward connectors and given gradients; outputs: the required gradients
            args = set(prog.arguments())
            assert args == set(lb.forward_inputs) | set(lb.forward_outputs) | set(lb.given_grad_names.values()) | \
                set(lb.required_grad_names.values()) | set(prog.constants)
            assert set(lb.forward_inputs) <= set(node.in_connectors)
            assert set(lb.forward_outputs) <= set(node.out_connectors)
            written = {a for t in prog.tasklets for a in t.outputs.values()}
            assert set(lb.required_grad_names.values()) <= written
            assert not written & (set(lb.forward_inputs) | set(lb.forward_outputs) | set(lb.given_grad_names.values()))
            for spec in prog.tasklets:
                functions.append(_tasklet_function(n, spec, prog))
                n += 1
    assert {"Einsum", "Softmax", "Add", "Sub", "Mul", "Div", "Pow", "Sqrt", "Erf", "ReduceMean", "Transpose", "Conv",
            "Sigmoid", "GlobalAveragePool", "Tanh", "Relu", "Exp", "Log", "Reciprocal"} <= ops
    _compile("".join(functions), tmp_path, "reverse_tasklets")
    # a softmax reverse reads the forward OUTPUT (torch's save_for_backward, autodiff/utils.py:224-261)
    g = graphs.GraphBuilder("sm", torch.float16)
    x = g.input("x", (8, 128))
    g.output(g.node("Softmax", {"input": x}, {"output": (8, 128)}, label="sm", axis=-1)["output"], "y")
    node = g.state.library_nodes()[0]
    lb = lowering.lower_backward(node, g.state, g.sdfg, find_backward_implementation(g.sdfg, g.state, node),
                                 ["output"], ["input"])
    assert lb.forward_outputs == ["output"] and lb.forward_inputs == []
    assert "dmlhip_softmax_backward_f16(_Y, _dY, _dX, 8, 128" in lb.program.tasklets[0].code()
    assert lb.program.tasklets[0].inputs == {"Y": "output", "dY": lb.given_grad_names["output"]}
    # a fused node whose reverse needs statistics the forward node would have to emit cannot stand alone
    g = graphs.GraphBuilder("ln", torch.float16)
    x = g.input("x", (8, 128))
    g.input("gamma", (128, ))
    g.input("beta", (128, ))
    g.output(g.layer_norm(x, "gamma", "beta", 1e-5, "ln"), "y")
    fusion.auto_optimize(g.sdfg)
    node = g.state.library_nodes()[0]
    with pytest.raises(NotApplicable):
        lowering.lower_backward(node, g.state, g.sdfg, find_backward_implementation(g.sdfg, g.state, node), ["Y"],
                                ["X", "Scale", "B"])


def test_stand_alone_reverse_programs_compute_what_the_in_graph_reverse_computes():
    """The reverse of a node lowered on its own (what DaCeML's generator would call through the registered
    BackwardImplementation, with arrays named after connectors) against the reverse the library's own generator builds
    inside the graph for the same node - both interpreted by tests/abi_emulator.py on the same values. The in-graph
    form is checked against the oracle by tests/test_emulated_graphs.py; this checks the plumbing around it: connector
    naming, copies for passed-through gradients, view offsets, constants."""
    from daceml_amd.runtime import expand_onnx_nodes
    from tests.abi_emulator import run_program, run_sdfg
    np_dtype = {torch.float16: np.float16, torch.float32: np.float32}
    samples = [graphs.bert_encoder_layer(2, 16, 64, 2, 128, torch.float32),
               graphs.mbconv_block(2, 16, 16, expand=2, cout=8, se_reduce=4, stride=2, dtype=torch.float32),
               _unary_graph(torch.float32, differentiable=True)]
    compared = set()
    for base in samples:
        count = len([x for x in base.states()[0].topological_sort() if isinstance(x, ONNXOp)])
        for i in range(count):
            sdfg = copy.deepcopy(base)
            st = sdfg.states()[0]
            node = [x for x in st.topological_sort() if isinstance(x, ONNXOp)][i]
            impl = find_backward_implementation(sdfg, st, node)
            given = [e.src_conn for e in st.out_edges(node)]
            required = [e.dst_conn for e in st.in_edges(node)
                        if e.data.data not in sdfg.constants and sdfg.arrays[e.data.data].dtype.is_floating_point]
            in_arr = {e.dst_conn: e.data.data for e in st.in_edges(node)}
            out_arr = {e.src_conn: e.data.data for e in st.out_edges(node)}
            if len(set(in_arr.values())) != len(in_arr):
                continue      # the same array on two connectors: the in-graph form sums the two gradients
            lb = lowering.lower_backward(node, st, sdfg, impl, given, required)

            # the same node alone in a graph of its own, reversed by the generator
            ref = copy.deepcopy(base)
            rst = ref.states()[0]
            rnode = [x for x in rst.topological_sort() if isinstance(x, ONNXOp)][i]
            for other in [x for x in rst.nodes() if isinstance(x, ONNXOp) and x is not rnode]:
                fusion._remove_node(rst, other)
            for name in list(in_arr.values()) + list(out_arr.values()):
                ref.arrays[name].transient = False
            grads = add_backward_pass(ref, rst, [out_arr[c] for c in given], [in_arr[c] for c in required])
            expand_onnx_nodes(ref)
            r = np.random.default_rng(100 + i)
            arrays = {}
            for c, name in in_arr.items():
                d = ref.arrays[name]
                if name not in ref.constants:
                    arrays[name] = r.uniform(0.5, 1.5, d.shape).astype(np_dtype[d.dtype])
            for c in given:
                d = ref.arrays[out_arr[c]]
                arrays["gradient_" + out_arr[c]] = r.standard_normal(d.shape).astype(np_dtype[d.dtype])
            run_sdfg(ref, arrays)

            mine = {}
            for c in lb.forward_inputs:
                mine[c] = arrays[in_arr[c]].copy()
            for c in lb.forward_outputs:
                mine[c] = arrays[out_arr[c]].copy()
            for c, name in lb.given_grad_names.items():
                mine[name] = arrays["gradient_" + out_arr[c]].copy()
            run_program(lb.program, mine)
            for c in required:
                got, want = mine[lb.required_grad_names[c]], arrays[grads[in_arr[c]]]
                assert got.shape == want.shape, (node, c)
                np.testing.assert_allclose(got, want, rtol=1e-6, atol=1e-7, err_msg="%s input %s" % (node, c))
            compared.add(node.schema.name)
    assert {"MatMul", "Softmax", "Add", "Sub", "Mul", "Div", "Pow", "Sqrt", "Erf", "ReduceMean", "Transpose", "Reshape",
            "Conv", "Sigmoid", "GlobalAveragePool", "Tanh", "Relu", "Exp", "Log", "Reciprocal"} <= compared, compared


def test_lowered_states_compute_what_the_runtime_computes():
    """A fused training graph (views in place of Transpose / Reshape nodes, grouped and K-concatenated contractions,
    fused attention) lowered state by state to TaskletPrograms - what is emitted as C++ - and interpreted, against
    the same expanded graph interpreted in the runtime's order: identical bits in every output."""
    from daceml_amd.runtime import expand_onnx_nodes
    from tests.abi_emulator import run_program, run_sdfg
    sdfg = graphs.bert_encoder_layer(2, 64, 128, 2, 256, torch.float16)
    fusion.auto_optimize(sdfg, training=True)
    add_backward_pass(sdfg, sdfg.states()[0], ["y"], ["x"] + graphs.BERT_PARAM_NAMES,
                      grad_dtypes={n: torch.float32 for n in graphs.BERT_PARAM_NAMES})
    fusion.optimize_backward(sdfg)
    expand_onnx_nodes(sdfg)
    assert any(d.view_of is not None for d in sdfg.arrays.values())
    r = np.random.default_rng(3)
    p = graphs.bert_init_params(128, 256, 5, bias_std=0.02)
    base = {n: p[n].astype(np.float16) for n in graphs.BERT_PARAM_NAMES}
    base["x"] = r.standard_normal((2, 64, 128)).astype(np.float16)
    base["gradient_y"] = r.standard_normal((2, 64, 128)).astype(np.float16)
    ref = {k: v.copy() for k, v in base.items()}
    run_sdfg(sdfg, ref)
    got = {k: v.copy() for k, v in base.items()}
    for st in sdfg.states():
        run_program(lowering.lower_state(sdfg, st), got)
    for name in ["y", "gradient_x"] + ["gradient_" + n for n in graphs.BERT_PARAM_NAMES]:
        assert np.array_equal(got[name], ref[name]), name


def test_emitted_program_runs_the_calls_in_dependency_order():
    sdfg = graphs.bert_encoder_layer(2, 64, 256, 4, 512, torch.float16)
    fusion.auto_optimize(sdfg)
    expand_onnx_nodes(sdfg)
    program = lowering.lower_state(sdfg, sdfg.states()[0])
    assert program.arguments()[0] == "x" and "y" in program.arguments()
    produced = set(program.arguments())
    for t in program.tasklets:
        assert set(t.inputs.values()) <= produced, "%s reads an array nothing has produced yet" % t.label
        produced |= set(t.outputs.values())
    text = lowering.emit_cxx(program, function="bert_forward")
    assert text.count("if (int __dml_status = ") == sum(len(t.calls) for t in program.tasklets)
    assert 'extern "C" int bert_forward(void* const* arguments, void* const* transients, void* workspace' in text
    # views are addressed through the array they alias: no array of the program is a view
    assert all(d.view_of is None for d in program.arrays.values())


# ----------------------------------------------------------------------------- install() against stand-ins
class _Recorder:
    """Stand-ins for the few DaCe / DaCeML entry points install() touches. They record what they are given."""
    def __init__(self, upstream=("Softmax", "Einsum", "MatMul", "Gemm", "Add", "Mul", "Conv", "Transpose", "Relu",
                                 "ReduceSum")):
        self.upstream = upstream
        self.forward_registry = {}
        self.node_implementations = {}
        self.backward_registry = {}

    def modules(self):
        rec = self
        from daceml_amd import sdfg as S

        class FakeState(S.SDFGState):
            def add_tasklet(self, label, ins, outs, code, language):
                t = S.Node(label)
                t.code, t.language, t.environments = code, language, set()
                for c in ins:
                    t.add_in_connector(c)
                for c in outs:
                    t.add_out_connector(c)
                return self.add_node(t)

            def add_nested_sdfg(self, nsdfg, parent, inputs, outputs):
                n = S.Node(nsdfg.name)
                n.sdfg = nsdfg
                for c in inputs:
                    n.add_in_connector(c)
                for c in outputs:
                    n.add_out_connector(c)
                return self.add_node(n)

        class FakeSDFG(S.SDFG):
            def add_array(self, name, shape, dtype, transient=False, strides=None, storage=None, find_new_name=False):
                return super().add_array(name, shape, dtype, transient=transient, strides=strides)

            def add_state(self, label=None):
                st = FakeState(label or "state_%d" % len(self._states), self)
                self._states.append(st)
                return st

            def nodes(self):
                return self.states()

        dace = types.ModuleType("dace")
        dace.SDFG = FakeSDFG
        for n in ("float16", "float32", "float64", "int64", "int32", "bool", "uint8"):
            setattr(dace, n, getattr(torch, n))      # descriptors of the stand-in SDFG carry torch dtypes
        dace.pointer = lambda t: ("pointer", t)
        dace.StorageType = types.SimpleNamespace(GPU_Global="GPU_Global")
        dace.dtypes = types.SimpleNamespace(Language=types.SimpleNamespace(CPP="CPP"))
        class LibraryNode(S.Node):
            def __init__(self, name, inputs=(), outputs=()):
                super().__init__(name)
                for c in inputs:
                    self.add_in_connector(c)
                for c in outputs:
                    self.add_out_connector(c)
        dace.nodes = types.SimpleNamespace(AccessNode=S.AccessNode, LibraryNode=LibraryNode)
        properties = types.ModuleType("dace.properties")
        properties.Property = lambda dtype=None, default=None, desc="": default
        dace.properties = properties
        library = types.ModuleType("dace.library")
        library.node = lambda cls: cls
        library.expansion = lambda cls: cls

        def environment(cls):
            cls.full_class_path = classmethod(lambda c: "daceml_amd.dace_plugin." + c.__name__)
            return cls
        library.environment = environment
        dace.library = library
        registry = types.ModuleType("dace.registry")

        def autoregister_params(**params):
            def dec(cls):
                rec.backward_registry[params.get("op") or params["node_type"]] = (cls, params)
                return cls
            return dec
        registry.autoregister_params = autoregister_params
        dace.registry = registry
        transformation = types.ModuleType("dace.transformation")
        tt = types.ModuleType("dace.transformation.transformation")
        tt.ExpandTransformation = type("ExpandTransformation", (), {})
        transformation.transformation = tt
        dace.transformation = transformation

        import daceml_amd.onnx as our
        daceml = types.ModuleType("daceml")
        donnx = types.ModuleType("daceml.onnx")
        upstream = set(rec.upstream)
        donnx.has_onnx_node = lambda name: name in upstream

        def node_class(op):
            class Cls(our.get_onnx_node(op)):       # instantiable like DaCeML's: ONNX<Op>(label, **attributes)
                implementations = {}

                @classmethod
                def register_implementation(cls, name, expansion):
                    rec.node_implementations.setdefault(op, {})[name] = expansion
            Cls.__name__ = "ONNX" + op
            return Cls
        for op in upstream:
            setattr(donnx, "ONNX" + op, node_class(op))
        daceml.onnx = donnx
        fia = types.ModuleType("daceml.onnx.forward_implementation_abc")
        fia.ONNXForward = type("ONNXForward", (), {})
        opi = types.ModuleType("daceml.onnx.op_implementations")
        opu = types.ModuleType("daceml.onnx.op_implementations.utils")

        def op_implementation(op, name):
            def dec(cls):
                rec.forward_registry[op] = (cls, name)
                return cls
            return dec
        opu.op_implementation = op_implementation
        util = types.ModuleType("daceml.util")
        uu = types.ModuleType("daceml.util.utils")
        uu.in_desc_with_name = S.in_desc_with_name
        uu.out_desc_with_name = S.out_desc_with_name
        nodes_pkg = types.ModuleType("daceml.onnx.nodes")
        onnx_op = types.ModuleType("daceml.onnx.nodes.onnx_op")
        onnx_op.ONNXOp = ONNXOp
        autodiff = types.ModuleType("daceml.autodiff")
        base_abc = types.ModuleType("daceml.autodiff.base_abc")
        base_abc.BackwardImplementation = type("BackwardImplementation", (), {})

        class BackwardResult:
            def __init__(self, required_grad_names, given_grad_names, zero_init=None):
                self.required_grad_names, self.given_grad_names = required_grad_names, given_grad_names
                self.zero_init = zero_init or {}
        base_abc.BackwardResult = BackwardResult
        butils = types.ModuleType("daceml.autodiff.utils")
        butils.forward_in_desc_with_name = lambda node, ctx, conn: S.in_desc_with_name(node, ctx.forward_state,
                                                                                        ctx.forward_sdfg, conn)
        butils.forward_out_desc_with_name = lambda node, ctx, conn: S.out_desc_with_name(node, ctx.forward_state,
                                                                                          ctx.forward_sdfg, conn)
        rec.forwarded = []
        butils.connect_output_from_forward = lambda fwd, bwd, ctx, conn: rec.forwarded.append((fwd.label, conn))
        return {"dace": dace, "dace.library": library, "dace.registry": registry, "dace.properties": properties,
                "dace.transformation": transformation,
                "dace.transformation.transformation": tt, "daceml": daceml, "daceml.onnx": donnx,
                "daceml.onnx.forward_implementation_abc": fia, "daceml.onnx.op_implementations": opi,
                "daceml.onnx.op_implementations.utils": opu, "daceml.util": util, "daceml.util.utils": uu,
                "daceml.onnx.nodes": nodes_pkg, "daceml.onnx.nodes.onnx_op": onnx_op, "daceml.autodiff": autodiff,
                "daceml.autodiff.base_abc": base_abc, "daceml.autodiff.utils": butils}, FakeSDFG


def test_install_registers_forward_and_backward_implementations(monkeypatch):
    from daceml_amd import dace_plugin
    import daceml_amd.onnx as our
    rec = _Recorder()
    mods, FakeSDFG = rec.modules()
    for name, mod in mods.items():
        monkeypatch.setitem(sys.modules, name, mod)
    registered = dace_plugin.install()
    assert sorted(registered["forward"]) == sorted(["Softmax", "Einsum", "MatMul", "Gemm", "Add", "Mul", "Conv",
                                                    "Transpose", "Relu", "ReduceSum"])
    assert sorted(registered["backward"]) == sorted(["Softmax", "Einsum", "MatMul", "Gemm", "Add", "Mul", "Conv",
                                                     "Transpose", "Relu", "ReduceSum"])
    # both registrations of the forward side (registry and node class)
    assert set(rec.forward_registry) == set(registered["forward"])
    assert all("hip" in rec.node_implementations[op] for op in registered["forward"])

    # a Softmax node on a stand-in "DaCe" SDFG expands to a nested SDFG: arrays named after the connectors, one C++
    # tasklet whose pointer connectors carry the underscore prefix, the environment attached
    s = FakeSDFG("outer")
    st = s.add_state()
    s.add_array("scores", (8, 16, 64, 64), torch.float16)
    s.add_array("probs", (8, 16, 64, 64), torch.float16)
    node = our.ONNXSoftmax("sm", axis=-1)
    st.add_edge(st.add_read("scores"), None, node, "input", s.make_array_memlet("scores"))
    st.add_edge(node, "output", st.add_write("probs"), None, s.make_array_memlet("probs"))
    expansion = rec.node_implementations["Softmax"]["hip"]
    node.validate = lambda sdfg, state: None
    nsdfg = expansion.expansion(node, st, s)
    assert sorted(nsdfg.arrays) == ["input", "output"] and not any(d.transient for d in nsdfg.arrays.values())
    (tasklet, ) = nsdfg.states()[0].library_nodes()
    assert sorted(tasklet.in_connectors) == ["_input"] and sorted(tasklet.out_connectors) == ["_output"]
    assert tasklet.code.startswith("if (int __dml_status = dmlhip_softmax_f16(_input, _output, 8192, 64, "
                                   "(void*)__dace_current_stream))")
    assert "throw std::runtime_error" in tasklet.code
    assert tasklet.environments == {"daceml_amd.dace_plugin.DaceMLHip"}
    edges = nsdfg.states()[0].edges()
    assert {(e.data.data, e.dst_conn) for e in edges if e.dst is tasklet} == {("input", "_input")}
    assert {(e.data.data, e.src_conn) for e in edges if e.src is tasklet} == {("output", "_output")}

    # its reverse node: a nested SDFG in the backward state, gradient connectors named by the BackwardResult, the
    # forward OUTPUT requested through connect_output_from_forward
    cls, params = rec.backward_registry["Softmax"]
    assert params == {"op": "Softmax", "name": "hip"} and cls.backward_can_be_applied(node, st, s)
    bst = s.add_state("backward")
    ctx = types.SimpleNamespace(forward_sdfg=s, forward_state=st, backward_sdfg=s, backward_state=bst,
                                backward_generator=None)
    rev, result = cls.backward(node, ctx, ["output"], ["input"])
    assert rev in bst.nodes() and rec.forwarded == [("sm", "output")]
    assert set(rev.in_connectors) == {"output", result.given_grad_names["output"]}
    assert set(rev.out_connectors) == {result.required_grad_names["input"]}
    assert result.zero_init == {result.required_grad_names["input"]: False}
    (t, ) = rev.sdfg.states()[0].library_nodes()
    assert "dmlhip_softmax_backward_f16" in t.code

    # an operand layout the kernels refuse (no dense inner dimension) is reported as not applicable, not raised
    s.add_array("strided", (8, 64), torch.float16, strides=(128, 2))
    s.add_array("out2", (8, 64), torch.float16)
    bad = our.ONNXSoftmax("sm2", axis=-1)
    st.add_edge(st.add_read("strided"), None, bad, "input", s.make_array_memlet("strided"))
    st.add_edge(bad, "output", st.add_write("out2"), None, s.make_array_memlet("out2"))
    assert rec.forward_registry["Softmax"][0].forward_can_be_applied(bad, st, s) is False


def test_training_graphs_reach_the_fused_kernels_as_library_nodes(monkeypatch):
    """What a ``post_onnx_hook`` of the reference's ``DaceModule(backward=True)`` does with ``fuse_for_training``: the
    decomposed BERT encoder layer is rewritten into fused nodes that are still LIBRARY nodes - DaCeML's own classes
    where it has one, one generic class otherwise - and each of them is given its "hip" reverse by the registry
    lookup the reference's backward-pass generator performs (find_backward_implementation, base_abc.py:114-159)."""
    from daceml_amd import dace_plugin, graphs
    opset12 = ("Softmax", "Einsum", "MatMul", "Gemm", "Add", "Sub", "Mul", "Div", "Pow", "Sqrt", "Erf", "ReduceMean",
               "Transpose", "Reshape", "Relu", "ReduceSum", "Identity", "Conv")
    rec = _Recorder(upstream=opset12)
    mods, FakeSDFG = rec.modules()
    for name, mod in mods.items():
        monkeypatch.setitem(sys.modules, name, mod)
    monkeypatch.setattr(dace_plugin, "_FUSED_NODE_CLASS", {})
    dace_plugin.install()

    # the reference's graph after import: opset-12 nodes only, on the stand-in "DaCe" classes
    sdfg = graphs.bert_encoder_layer(2, 64, 128, 2, 256, torch.float16, eps=1e-12)
    state = sdfg.states()[0]
    assert {n.schema.name for n in state.library_nodes()} <= set(opset12)
    n_before = len(state.library_nodes())
    sdfg.__class__ = FakeSDFG
    state.__class__ = type(FakeSDFG("x").add_state())
    # the reference's importer keeps the values of initialisers in ONNXModel.weights
    module = types.SimpleNamespace(sdfg=sdfg, backward=True,
                                   dace_model=types.SimpleNamespace(weights=dict(sdfg.constants)))
    assert dace_plugin.fuse_for_training(module) == 1

    fused_cls = dace_plugin.make_fused_node_class(mods["dace"])
    nodes = [n for n in state.nodes() if not isinstance(n, mods["dace"].nodes.AccessNode)]
    assert len(nodes) < n_before
    kinds = {}
    for n in nodes:
        if isinstance(n, fused_cls):
            kinds.setdefault(n.hip_kind, []).append(n)
        else:
            assert n.schema.name in opset12 and type(n).__name__ == "ONNX" + n.schema.name
    assert len(kinds["LayerNormalization"]) == 2 and len(kinds["FusedAttention"]) == 1 and "FusedEinsum" in kinds
    assert any(k in kinds for k in ("Gelu", "BiasGelu")) and "Softmax" not in {getattr(n, "schema", None) and
                                                                                 n.schema.name for n in nodes}
    # created with the outputs their reverse nodes will ask for
    ln = kinds["LayerNormalization"][0]
    assert {"Mean", "InvStdDev"} <= set(ln.out_connectors)
    assert "LogSumExp" in kinds["FusedAttention"][0].out_connectors
    # ... and the rewritten state still computes the layer: its forward expansions lower to the kernels' entry points
    expand = fused_cls.implementations["hip"].expansion
    assert "dmlhip_layernorm_f16" in expand(ln, state, sdfg).states()[0].library_nodes()[0].code
    att = kinds["FusedAttention"][0]
    assert "dmlhip_attention_f16" in expand(att, state, sdfg).states()[0].library_nodes()[0].code

    # the generator's lookup: by node class for the fused nodes
    cls, params = rec.backward_registry[fused_cls]
    assert params == {"node_type": fused_cls, "name": "hip"}
    bst = sdfg.add_state("backward")
    ctx = types.SimpleNamespace(forward_sdfg=sdfg, forward_state=state, backward_sdfg=sdfg, backward_state=bst,
                                backward_generator=None)
    # (LayerNormalization: the scale / shift gradients have the parameters' fp16 under the reference)
    expected = {"LayerNormalization": "dmlhip_layernorm_backward_grads_f16", "FusedAttention": "dmlhip_attention_backward_f16",
                "Gelu": "dmlhip_unary_backward_f16", "BiasGelu": "dmlhip_", "FusedEinsum": "dmlhip_gemm_f16"}
    for kind, members in kinds.items():
        node = members[0]
        assert cls.backward_can_be_applied(node, state, sdfg), kind
        given = [e.src_conn for e in state.out_edges(node) if e.src_conn in ("Y", "Output", "output")]
        required = [e.dst_conn for e in state.in_edges(node) if e.dst_conn not in ("Mask", )]
        rec.forwarded.clear()
        rev, result = cls.backward(node, ctx, given, required)
        code = "\n".join(t.code for t in rev.sdfg.states()[0].library_nodes())
        assert expected[kind] in code, (kind, code[:300])
        assert set(result.required_grad_names) == set(required)
        if kind == "LayerNormalization":    # the statistics come from the forward node, not from a recomputation
            assert {c for _, c in rec.forwarded} >= {"Mean", "InvStdDev"}
        if kind == "FusedAttention":
            assert {c for _, c in rec.forwarded} >= {"Output", "LogSumExp"}
