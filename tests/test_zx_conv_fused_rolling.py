"""The rolling-window form of the fused pointwise + depthwise convolution (what the library runs; its geometry pinned
through ``dmlhip_debug_fused_rolling``) on the problems the strip kernel is tested with, and on the benchmarked MBConv shape,
where it must agree with the strip kernel bit for bit (both add in the same order).
"""
import numpy as np
import pytest
import torch

from oracle import ops as O
from tests import test_gpu_kernels as TK
from tests.util import assert_close, dev, host

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("waves", [8, 16])
@pytest.mark.parametrize("n,cin,cmid,h,w,stride,acts,has_bias", TK.EXPAND_DEPTHWISE_CASES)
def test_conv2d_expand_depthwise_rolling(n, cin, cmid, h, w, stride, acts, has_bias, waves):
    from daceml_amd import _lib as L, kernels as K
    code = {"none": L.ACT_NONE, "swish": L.ACT_SWISH, "relu": L.ACT_RELU}
    fn = {"none": lambda t: t, "swish": O.swish, "relu": lambda t: np.maximum(t, 0.0)}
    r = np.random.default_rng(140)
    x = r.standard_normal((n, cin, h, w)).astype(np.float32)
    w1 = (r.standard_normal((cmid, cin, 1, 1)) * np.sqrt(2.0 / cin)).astype(np.float32)
    w2 = (r.standard_normal((cmid, 1, 3, 3)) * np.sqrt(2.0 / 9)).astype(np.float32)
    b1 = (r.standard_normal(cmid) * 0.1).astype(np.float32) if has_bias else None
    b2 = (r.standard_normal(cmid) * 0.1).astype(np.float32) if has_bias else None
    f64 = lambda t: None if t is None else t.astype(np.float64)  # noqa: E731
    mid = fn[acts[0]](O.conv2d(f64(x), f64(w1), f64(b1)))
    want = fn[acts[1]](O.conv2d(mid, f64(w2), f64(b2), (stride, stride), (1, 1, 1, 1), (1, 1), cmid))
    lib = L.load()
    run = lambda: K.conv2d_expand_depthwise(dev(x), dev(w1), None if b1 is None else dev(b1), dev(w2),  # noqa: E731
                                            None if b2 is None else dev(b2), stride=stride, act_pw=code[acts[0]],
                                            act_dw=code[acts[1]])
    lib.dmlhip_debug_fused_rolling(-2, 8)
    strips = host(run())
    try:
        for rows in (0, -1, 1, 2):
            lib.dmlhip_debug_fused_rolling(rows, waves)
            got = host(run())
            assert_close(got, want, torch.float32, "rolling window, rows %d" % rows, rtol=1e-5, atol=4e-6)
            assert np.array_equal(got, strips), "rows %d: differs from the strip kernel" % rows
    finally:
        lib.dmlhip_debug_fused_rolling(0, 8)


@pytest.mark.parametrize("waves", [8, 16])
def test_rolling_window_on_the_benchmarked_block(waves):
    """[96,32,112,112] -> 192 channels, stride 2, swish / swish: 2304 workgroups of 7 batches; against the strip kernel
    (itself checked against the oracle at this size in tests/test_gpu_fullsize.py)."""
    from daceml_amd import _lib as L, kernels as K
    g = torch.Generator(device="cpu").manual_seed(5)
    x = torch.randn((96, 32, 112, 112), generator=g).cuda()
    w1 = (torch.randn((192, 32, 1, 1), generator=g) * 0.25).cuda()
    b1 = (torch.randn(192, generator=g) * 0.1).cuda()
    w2 = (torch.randn((192, 1, 3, 3), generator=g) * 0.47).cuda()
    b2 = (torch.randn(192, generator=g) * 0.1).cuda()
    lib = L.load()
    run = lambda: K.conv2d_expand_depthwise(x, w1, b1, w2, b2, stride=2, act_pw=L.ACT_SWISH, act_dw=L.ACT_SWISH)  # noqa: E731
    lib.dmlhip_debug_fused_rolling(-2, 8)
    strips = run()
    try:
        lib.dmlhip_debug_fused_rolling(-1, waves)
        got = run()
        lib.dmlhip_debug_fused_rolling(0, waves)
        chosen = run()
        torch.cuda.synchronize()
    finally:
        lib.dmlhip_debug_fused_rolling(0, 8)
    assert got.shape == strips.shape == (96, 192, 56, 56)
    assert torch.equal(got, strips) and torch.equal(chosen, strips)
