"""Conv nodes whose X and / or Y are channels-last: shape in ONNX order [N, C, H, W], strides of a dense [N, H, W, C]
tensor - the layout ``_get_tensor_layout`` detects and hands to cuDNN as CUDNN_TENSOR_NHWC
(cudnn_implementations.py:20-110). Here such an operand passes through a transpose into / out of the workspace around
the NCHW kernels. Oracle: ``oracle.ops.conv2d`` on the logical tensors.

Host side: the emitted calls interpreted by tests/abi_emulator.py on the operands' memory images. GPU: the same
graphs run on torch tensors in ``torch.channels_last`` memory format (which has exactly these strides)."""
import numpy as np
import pytest
import torch

from oracle import ops as O
from tests.util import assert_close, dev, host, rng

# n, c, h, w, m, k, stride, pad, group, x channels-last, y channels-last
CASES = [(2, 8, 12, 14, 16, 3, 1, 1, 1, True, True), (2, 8, 12, 14, 16, 3, 2, 1, 1, True, False),
         (3, 6, 9, 9, 6, 3, 1, 1, 6, False, True), (2, 32, 10, 10, 48, 1, 1, 0, 1, True, True),
         (1, 4, 7, 5, 8, 5, 1, 2, 2, True, True)]


def _nhwc_strides(shape):
    n, c, h, w = shape
    return (h * w * c, 1, w * c, c)


def _case(dtype, n, c, h, w, m, k, stride, pad, group, x_last, y_last):
    from daceml_amd import graphs
    npdt = np.float16 if dtype == torch.float16 else np.float32
    r = rng(71)
    x = r.standard_normal((n, c, h, w)).astype(npdt)
    wt = (r.standard_normal((m, c // group, k, k)) / np.sqrt(c // group * k * k)).astype(npdt)
    b = r.standard_normal(m).astype(npdt)
    want = O.conv2d(x.astype(np.float64), wt.astype(np.float64), b.astype(np.float64), (stride, stride), (pad, ) * 4, (1, 1),
                    group)
    g = graphs.GraphBuilder("conv_layouts", dtype)
    g.sdfg.add_array("x", x.shape, dtype, strides=_nhwc_strides(x.shape) if x_last else None)
    ins = {"X": "x", "W": g.input("w", wt.shape), "B": g.input("b", (m, ))}
    y = g.node("Conv", ins, {"Y": want.shape}, label="conv", kernel_shape=[k, k], strides=[stride, stride],
               pads=[pad] * 4, group=group)["Y"]
    g.output(y, "y")
    if y_last:
        g.sdfg.arrays["y"].strides = _nhwc_strides(want.shape)
    return g, x, wt, b, want


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("case", CASES)
def test_channels_last_operands_lower_to_transposes_around_the_kernel(case, dtype):
    from daceml_amd.runtime import expand_onnx_nodes
    from tests.abi_emulator import run_state
    x_last, y_last = case[-2:]
    g, x, wt, b, want = _case(dtype, *case)
    expand_onnx_nodes(g.sdfg)
    tasklet = g.state.library_nodes()[0]
    sfx = "f16" if dtype == torch.float16 else "f32"
    assert [c.symbol for c in tasklet.calls] == (["dmlhip_transpose_" + sfx] if x_last else []) + ["dmlhip_conv2d_" + sfx] + \
        (["dmlhip_transpose_" + sfx] if y_last else [])
    item = 2 if dtype == torch.float16 else 4
    need = (x.size * item + 255) // 256 * 256 * x_last + (want.size * item + 255) // 256 * 256 * y_last
    assert tasklet.workspace_bytes == need
    # the arrays as they lie in memory
    arrays = {"x": np.ascontiguousarray(x.transpose(0, 2, 3, 1)) if x_last else x.copy(), "w": wt.copy(), "b": b.copy()}
    run_state(g.sdfg, g.state, arrays)
    got = arrays["y"].reshape(-1)
    n, m, oh, ow = want.shape
    got = got.reshape(n, oh, ow, m).transpose(0, 3, 1, 2) if y_last else got.reshape(want.shape)
    tol = dict(rtol=1e-5, atol=2e-6) if dtype == torch.float32 else dict(rtol=2e-2, atol=1e-2)
    assert_close(got, want, dtype, "emulated conv %s" % (case, ), **tol)


def test_layout_detection_follows_the_reference():
    """``_get_tensor_layout`` (cudnn_implementations.py:20-66): dense -> NCHW; channels-last strides -> NHWC; anything
    else -> no layout, and the node is refused."""
    import daceml_amd.onnx as donnx
    from daceml_amd.onnx.op_implementations.hip_implementations import _tensor_layout
    from daceml_amd.sdfg import Array
    assert _tensor_layout(Array((2, 3, 4, 5), torch.float32, False, None)) == "NCHW"
    assert _tensor_layout(Array((2, 3, 4, 5), torch.float32, False, (60, 1, 15, 3))) == "NHWC"
    assert _tensor_layout(Array((2, 3, 7), torch.float32, False, (21, 1, 3))) == "NHWC"
    assert _tensor_layout(Array((2, 3, 4, 5), torch.float32, False, (120, 20, 5, 1))) is None      # padded rows
    assert _tensor_layout(Array((2, 3, 4, 5), torch.float32, False, (60, 5, 15, 1))) is None       # some other permutation
    assert _tensor_layout(Array((2, 1, 4, 5), torch.float32, False, None)) == "NCHW"                # one channel: the same bytes
    g, *_ = _case(torch.float32, 2, 8, 12, 14, 16, 3, 1, 1, 1, False, False)
    g.sdfg.arrays["x"].strides = (8 * 12 * 16, 12 * 16, 16, 1)
    with pytest.raises(donnx.NotApplicable):
        g.state.library_nodes()[0].expand(g.sdfg, g.state)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("case", CASES)
def test_channels_last_conv_on_gpu(case, dtype):
    from daceml_amd.runtime import CompiledSDFG
    x_last, y_last = case[-2:]
    g, x, wt, b, want = _case(dtype, *case)
    prog = CompiledSDFG(g.sdfg)
    xt = dev(x).contiguous(memory_format=torch.channels_last) if x_last else dev(x)
    y = torch.full(want.shape, float("nan"), dtype=dtype, device="cuda")
    if y_last:
        y = y.contiguous(memory_format=torch.channels_last)
    assert not x_last or tuple(xt.stride()) == _nhwc_strides(x.shape)
    prog(x=xt, w=dev(wt), b=dev(b), y=y)
    tol = dict(rtol=1e-5, atol=2e-6) if dtype == torch.float32 else dict(rtol=2e-2, atol=1e-2)
    assert_close(host(y), want, dtype, "channels-last conv %s" % (case, ), **tol)
    assert np.array_equal(host(xt), x.astype(np.float32) if dtype == torch.float16 else x), "X is read-only"
