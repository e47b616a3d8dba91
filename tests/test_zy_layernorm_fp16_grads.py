"""LayerNormalization in a training graph without fp32 master gradients: the scale / shift gradients have the dtype of
their forward arrays (as every gradient has under the reference, backward_pass_generator.py:642-700), while the kernel
sums them in fp32 and rounds them once as it stores them (``dmlhip_layernorm_backward_grads_f16``). Host side: the calls are
interpreted by tests/abi_emulator.py; GPU: the kernels. Oracle: ``oracle.ops.layernorm_backward``."""
import numpy as np
import pytest
import torch

from oracle import ops as O
from tests.util import assert_close, dev, host


def _layernorm_training_graph():
    from daceml_amd import graphs
    from daceml_amd.autodiff import add_backward_pass
    from daceml_amd.transformation import fusion
    g = graphs.GraphBuilder("ln_train", torch.float16)
    xin = g.input("x", (6, 40, 256))
    g.input("gamma", (256, ))
    g.input("beta", (256, ))
    g.output(g.layer_norm(xin, "gamma", "beta", 1e-5, "ln"), "y")
    fusion.auto_optimize(g.sdfg, training=True)
    # no fp32 master gradients asked for: as under the reference, a gradient has the dtype of its forward array
    grads = add_backward_pass(g.sdfg, g.state, ["y"], ["x", "gamma", "beta"])
    assert g.sdfg.arrays[grads["gamma"]].dtype == torch.float16 and g.sdfg.arrays[grads["beta"]].dtype == torch.float16
    return g.sdfg


def _layernorm_training_data():
    r = np.random.default_rng(77)
    x = r.standard_normal((6, 40, 256)).astype(np.float16)
    dy = r.standard_normal((6, 40, 256)).astype(np.float16)
    gamma = r.uniform(0.5, 1.5, 256).astype(np.float16)
    beta = (r.standard_normal(256) * 0.1).astype(np.float16)
    want = O.layernorm_backward(dy.astype(np.float64), x.astype(np.float64), gamma.astype(np.float64), 1e-5)
    return x, dy, gamma, beta, want


def _check_layernorm_gradients(dx, dg, db, want):
    assert_close(dx, want[0], torch.float16, "dx")
    # sums of 240 exact fp16 products in fp32, rounded once to fp16: the stated tolerance as it stands
    assert_close(dg, want[1], torch.float16, "dgamma")
    assert_close(db, want[2], torch.float16, "dbeta")


def test_layernorm_scale_and_shift_gradients_in_fp16_lower_correctly():
    """One call, no casts, when the graph wants fp16 gradients."""
    from daceml_amd.runtime import expand_onnx_nodes
    from tests.abi_emulator import run_sdfg
    sdfg = _layernorm_training_graph()
    expand_onnx_nodes(sdfg)
    calls = [c.symbol for st in sdfg.states() for n in st.nodes() for c in (getattr(n, "calls", None) or [])]
    assert "dmlhip_cast" not in calls and "dmlhip_layernorm_backward_grads_f16" in calls
    x, dy, gamma, beta, want = _layernorm_training_data()
    arrays = {"x": x.copy(), "gamma": gamma.copy(), "beta": beta.copy(), "gradient_y": dy.copy()}
    run_sdfg(sdfg, arrays)
    _check_layernorm_gradients(arrays["gradient_x"], arrays["gradient_gamma"], arrays["gradient_beta"], want)


@pytest.mark.gpu
def test_layernorm_scale_and_shift_gradients_in_fp16_on_gpu():
    from daceml_amd.runtime import CompiledSDFG
    prog = CompiledSDFG(_layernorm_training_graph())
    x, dy, gamma, beta, want = _layernorm_training_data()
    out = {n: torch.full(s, float("nan"), dtype=torch.float16, device="cuda")
           for n, s in (("y", x.shape), ("gradient_x", x.shape), ("gradient_gamma", (256, )), ("gradient_beta", (256, )))}
    prog(x=dev(x), gamma=dev(gamma), beta=dev(beta), gradient_y=dev(dy), **out)
    _check_layernorm_gradients(host(out["gradient_x"]), host(out["gradient_gamma"]), host(out["gradient_beta"]), want)
