"""The committed fixtures (tests/golden/hot_ops.npz, written by tests/golden/make_fixtures.py) against the oracle on
the CPU and against the HIP kernels on the GPU."""
import os

import numpy as np
import pytest
import torch

from oracle import ops as O
from tests.util import assert_close, dev, host

HERE = os.path.dirname(os.path.abspath(__file__))
FIX = np.load(os.path.join(HERE, "golden", "hot_ops.npz"))


def test_fixture_file_is_what_the_generator_writes():
    import importlib.util
    spec = importlib.util.spec_from_file_location("make_fixtures", os.path.join(HERE, "golden", "make_fixtures.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    fresh = mod.build()
    assert sorted(fresh) == sorted(FIX.files)
    for k in FIX.files:
        np.testing.assert_allclose(fresh[k], FIX[k], rtol=1e-12, atol=1e-13, err_msg=k)


def test_oracle_reproduces_fixtures_and_reference_literal():
    # tests/test_onnx_return_scalars.py:43-46 of the reference: ReduceSum over [1, 2, 3, 4] is 10
    assert O.reduce_sum(FIX["reducesum_literal_in"], [0], 0) == FIX["reducesum_literal_out"] == 10.0
    np.testing.assert_allclose(O.softmax(FIX["softmax_x"], 1), FIX["softmax_y"], rtol=1e-13)
    np.testing.assert_allclose(O.gelu_chain(FIX["gelu_x"]), FIX["gelu_y"], rtol=1e-13, atol=1e-300)
    assert FIX["gelu_y"][60] == 0.0 and abs(FIX["gelu_y"][62] - 6.0) < 1e-8 and abs(FIX["gelu_y"][61]) < 1e-8
    assert FIX["conv_y"].shape == (5, 16, 4, 4)   # the shapes of examples/plot_conv.py:16-46
    np.testing.assert_allclose(O.conv2d_loops(FIX["conv_x"][:1], FIX["conv_w"][:2], None, strides=(2, 2)),
                               FIX["conv_y"][:1, :2], rtol=1e-12)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
def test_kernels_against_fixtures(dtype):
    from daceml_amd import _lib as L, kernels as K
    npdt = np.float32 if dtype == torch.float32 else np.float16

    def d(name):
        return dev(FIX[name].astype(npdt))

    def ref(fn, *names):
        # the kernels see inputs rounded to their element type: evaluate the oracle on the same values
        return fn(*[FIX[n].astype(npdt).astype(np.float64) for n in names])

    y = K.softmax(d("softmax_x"))
    assert_close(host(y), ref(lambda x: O.softmax(x, 1), "softmax_x"), dtype, "softmax")
    assert_close(host(K.softmax_backward(y, d("softmax_dy"))),
                 O.softmax_backward(host(y).astype(np.float64), FIX["softmax_dy"].astype(npdt).astype(np.float64), 1), dtype,
                 "softmax backward")
    assert_close(host(K.layernorm(d("ln_x"), d("ln_gamma"), d("ln_beta"), 1e-5)[0]),
                 ref(lambda x, g, b: O.layernorm_chain(x, g, b, 1e-5)[0], "ln_x", "ln_gamma", "ln_beta"), dtype, "layernorm")
    assert_close(host(K.unary(L.GELU, d("gelu_x"))), ref(O.gelu_chain, "gelu_x"), dtype, "gelu")
    assert_close(host(K.einsum("aik,kj->aij", d("matmul_a"), d("matmul_b"))), ref(O.matmul, "matmul_a", "matmul_b"), dtype,
                 "matmul", atol=None if dtype == torch.float16 else 4e-6)
    assert_close(host(K.reduce(L.RSUM, d("reduce_x"), [0, 1], False, out_dtype=torch.float32)),
                 ref(lambda x: O.reduce_sum(x, [0, 1], 0), "reduce_x"), torch.float32, "reduce_sum", atol=1e-5)
    y, om, ov, sm, sv = K.batchnorm_training(d("bn_x"), d("bn_scale"), d("bn_bias"), d("bn_mean"), d("bn_var"), 1e-5, 0.9)
    names = ("bn_x", "bn_scale", "bn_bias", "bn_mean", "bn_var")
    want = ref(lambda *a: O.batchnorm_training(*a, 1e-5, 0.9), *names)
    for got, w, what in zip((y, om, ov, sm, sv), want, ("y", "running mean", "running variance", "mean", "variance")):
        assert_close(host(got), w, dtype, "batchnorm " + what)
    assert_close(host(K.batchnorm_inference(*[d(n) for n in names], 1e-5)),
                 ref(lambda *a: O.batchnorm_inference(*a, 1e-5), *names), dtype, "batchnorm inference")
    if dtype == torch.float32:
        assert_close(host(K.conv2d(d("conv_x"), d("conv_w"), None, strides=(2, 2))), FIX["conv_y"], dtype, "conv C1",
                     rtol=1e-5, atol=1e-5)
        dx, dw = K.conv2d_backward(d("conv_x"), d("conv_w"), d("conv_dy"), (2, 2))
        assert_close(host(dx), FIX["conv_dx"], dtype, "conv C1 dx", rtol=1e-5, atol=1e-5)
        assert_close(host(dw), FIX["conv_dw"], dtype, "conv C1 dw", rtol=1e-5, atol=2e-5)
        dx, dsc, dbi = K.batchnorm_backward(d("bn_dy"), d("bn_x"), d("bn_scale"), d("bn_saved_mean"), d("bn_saved_var"), 1e-5)
        for got, name in ((dx, "bn_dx"), (dsc, "bn_dscale"), (dbi, "bn_dbias")):
            assert_close(host(got), FIX[name], dtype, name, rtol=1e-4, atol=1e-5)
        got = K.conv2d_expand_depthwise(d("mb_x"), d("mb_w1"), d("mb_b1"), d("mb_w2"), d("mb_b2"), stride=2,
                                        act_pw=L.ACT_SWISH, act_dw=L.ACT_SWISH)
        assert_close(host(got), FIX["mb_y"], dtype, "expand + depthwise", rtol=1e-5, atol=4e-6)
    else:
        out, lse = K.attention(d("attn_q"), d("attn_k"), d("attn_v"), 0.125)
        want, want_lse = ref(lambda q, k, v: O.attention(q, k, v, 0.125), "attn_q", "attn_k", "attn_v")
        assert_close(host(out), want, dtype, "attention")
        assert_close(host(lse), want_lse, torch.float32, "attention lse", rtol=1e-3, atol=1e-3)
        dq, dk, dv = K.attention_backward(d("attn_q"), d("attn_k"), d("attn_v"), out, lse, d("attn_do"), 0.125)
        wq, wk, wv = ref(lambda q, k, v, g: O.attention_backward(q, k, v, 0.125, g), "attn_q", "attn_k", "attn_v", "attn_do")
        for name, got, w in (("dq", dq, wq), ("dk", dk, wk), ("dv", dv, wv)):
            assert_close(host(got), w, dtype, "attention " + name, atol=1e-2 * max(1.0, float(np.abs(w).max())))
