"""Writes tests/golden/hot_ops.npz: seeded inputs and the oracle's outputs (fp64) for every operator on the path,
at sizes of a few hundred elements.

The reference's own tests hold no literal vectors for these operators (they compare against NumPy / PyTorch on
unseeded random inputs), so the fixtures freeze the *pinned* oracle (tests/test_oracle.py pins it against
torch / scipy / autograd / brute-force loops): a later edit of oracle/ that changes a result fails
tests/test_golden.py on the CPU, and the GPU parity tests check the kernels against the same frozen numbers.
The one literal the reference does hold on the path, ReduceSum([1,2,3,4]) == 10
(tests/test_onnx_return_scalars.py:43-46), is included. Conv uses the literal shapes of examples/plot_conv.py:16-46.

Run from the repo root:  python tests/golden/make_fixtures.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import ops as O  # noqa: E402


def build():
    r = np.random.default_rng(20240607)
    f = {}
    x = r.standard_normal((4, 37))
    f["softmax_x"], f["softmax_y"] = x, O.softmax(x, axis=1)
    dy = r.standard_normal((4, 37))
    f["softmax_dy"], f["softmax_dx"] = dy, O.softmax_backward(f["softmax_y"], dy, 1)
    x, g, b = r.standard_normal((3, 48)), r.uniform(0.5, 1.5, 48), r.standard_normal(48) * 0.1
    f["ln_x"], f["ln_gamma"], f["ln_beta"], f["ln_y"] = x, g, b, O.layernorm_chain(x, g, b, 1e-5)[0]
    dy = r.standard_normal((3, 48))
    dx, dg, db = O.layernorm_backward(dy, x, g, 1e-5)
    f["ln_dy"], f["ln_dx"], f["ln_dgamma"], f["ln_dbeta"] = dy, dx, dg, db
    x = np.concatenate([r.standard_normal(60) * 2, [0.0, -6.0, 6.0, 1e-4]])
    f["gelu_x"], f["gelu_y"] = x, O.gelu_chain(x)
    f["gelu_dy"] = r.standard_normal(64)
    f["gelu_dx"] = O.gelu_backward(f["gelu_dy"], x)
    a, bb = r.standard_normal((2, 8, 16)), r.standard_normal((16, 24))
    f["matmul_a"], f["matmul_b"], f["matmul_y"] = a, bb, O.matmul(a, bb)
    q, k, v = r.standard_normal((1, 2, 9, 64)), r.standard_normal((1, 2, 5, 64)), r.standard_normal((1, 2, 5, 64))
    out, lse = O.attention(q, k, v, 0.125)
    do = r.standard_normal((1, 2, 9, 64))
    dq, dk, dv = O.attention_backward(q, k, v, 0.125, do)
    f.update(attn_q=q, attn_k=k, attn_v=v, attn_out=out, attn_lse=lse, attn_do=do, attn_dq=dq, attn_dk=dk, attn_dv=dv)
    x, w = r.uniform(0, 1, (5, 3, 10, 10)), r.uniform(0, 1, (16, 3, 3, 3))
    f["conv_x"], f["conv_w"] = x, w
    f["conv_y"] = O.conv2d(x, w, None, strides=(2, 2))
    f["reducesum_literal_in"], f["reducesum_literal_out"] = np.array([1.0, 2.0, 3.0, 4.0]), np.array(10.0)
    f["reduce_x"] = r.standard_normal((6, 5, 8))
    f["reduce_sum_01"] = O.reduce_sum(f["reduce_x"], [0, 1], 0)
    f["reduce_mean_2"] = O.reduce_mean(f["reduce_x"], [2], 1)
    # later additions draw after everything above, so the earlier vectors keep their values
    x = r.standard_normal((4, 3, 5, 6)) * 2 + 1
    sc, bi = r.uniform(0.5, 1.5, 3), r.standard_normal(3) * 0.1
    rm, rv = r.standard_normal(3) * 0.2, r.uniform(0.5, 1.5, 3)
    y, om, ov, sm, sv = O.batchnorm_training(x, sc, bi, rm, rv, 1e-5, 0.9)
    dy = r.standard_normal(x.shape)
    dx, dsc, dbi = O.batchnorm_backward(dy, x, sc, sm, sv, 1e-5)
    f.update(bn_x=x, bn_scale=sc, bn_bias=bi, bn_mean=rm, bn_var=rv, bn_y=y, bn_out_mean=om, bn_out_var=ov,
             bn_saved_mean=sm, bn_saved_var=sv, bn_dy=dy, bn_dx=dx, bn_dscale=dsc, bn_dbias=dbi,
             bn_y_inference=O.batchnorm_inference(x, sc, bi, rm, rv, 1e-5))
    dy = r.standard_normal(f["conv_y"].shape)
    dx, dw, _ = O.conv2d_backward(f["conv_x"], f["conv_w"], dy, strides=(2, 2))
    f.update(conv_dy=dy, conv_dx=dx, conv_dw=dw)
    # the expand + depthwise stages of an MBConv block: 1x1 conv + swish, then 3x3 depthwise stride 2 pad 1 + swish
    x = r.standard_normal((1, 16, 6, 7))
    w1, b1 = r.standard_normal((32, 16, 1, 1)) * 0.35, r.standard_normal(32) * 0.1
    w2, b2 = r.standard_normal((32, 1, 3, 3)) * 0.45, r.standard_normal(32) * 0.1
    mid = O.swish(O.conv2d(x, w1, b1))
    f.update(mb_x=x, mb_w1=w1, mb_b1=b1, mb_w2=w2, mb_b2=b2,
             mb_y=O.swish(O.conv2d(mid, w2, b2, (2, 2), (1, 1, 1, 1), (1, 1), 32)))
    return f


if __name__ == "__main__":
    out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "hot_ops.npz")
    np.savez_compressed(out, **build())
    print(out, os.path.getsize(out), "bytes")
