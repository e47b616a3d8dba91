"""A NumPy interpreter for a few entry points of include/daceml_hip.h, written from the header's comments.

TEST INFRASTRUCTURE ONLY. It lets the host-side tests check what an expansion ASKS the library to do (descriptor
contents, operand order, workspace use, the sequence of calls) on a machine without a GPU: an expansion's
``HipCall``s are run against NumPy arrays and the result is compared with the oracle. It says nothing about the
kernels themselves; those are checked on the GPU against the same oracle.
"""
import math

import numpy as np
from numpy.lib.stride_tricks import as_strided

from daceml_amd import _lib as L
from daceml_amd import hip_tasklet as T


def _view(buf, offset, shape, strides):
    """Strided view (element strides) into the flat array `buf`."""
    item = buf.itemsize
    flat = buf.reshape(-1)
    return as_strided(flat[offset:], shape=shape, strides=[s * item for s in strides], writeable=False)


def _act(kind, v):
    if kind == L.ACT_NONE:
        return v
    if kind == L.ACT_GELU:
        from scipy.special import erf
        return 0.5 * v * (1.0 + erf(v / math.sqrt(2.0)))
    if kind == L.ACT_RELU:
        return np.maximum(v, 0)
    if kind == L.ACT_SIGMOID:
        return 1 / (1 + np.exp(-v))
    if kind == L.ACT_SWISH:
        return v / (1 + np.exp(-v))
    raise ValueError(kind)


def gemm(desc, a, b, c, bias, residual, pre_out):
    """dmlhip_gemm_*: C[b][m, n] = act(alpha * sum_k A[b][m, k] B[b][k, n] + bias) + residual + beta * C. `a`, `b`,
    `c`, ... are flat arrays; fp32 accumulation, one rounding to C's type."""
    m, n, k = desc.m, desc.n, desc.k
    batch = tuple(desc.batch)
    av = _view(a, 0, batch + (m, k), tuple(desc.a_stride_batch) + (desc.a_stride_m, desc.a_stride_k))
    bv = _view(b, 0, batch + (k, n), tuple(desc.b_stride_batch) + (desc.b_stride_k, desc.b_stride_n))
    acc = np.matmul(av.astype(np.float64), bv.astype(np.float64)) * float(desc.alpha)
    if bias is not None:
        bb = bias.reshape(-1).astype(np.float64)
        acc = acc + (bb[:m].reshape(m, 1) if desc.bias_along_m else bb[:n].reshape(1, n))
    cs = tuple(desc.c_stride_batch) + (desc.c_stride_m, 1)
    out_dtype = np.float16 if desc.out_dtype == L.F16 else np.float32
    if c.dtype != out_dtype:
        raise TypeError("C has dtype %s, the descriptor says %s" % (c.dtype, out_dtype))
    if pre_out is not None:
        pv = as_strided(pre_out.reshape(-1), shape=batch + (m, n), strides=[s * pre_out.itemsize for s in cs])
        pv[...] = acc.astype(out_dtype)
        acc = pv.astype(np.float64)
    acc = _act(desc.act, acc)
    if residual is not None:
        acc = acc + _view(residual, 0, batch + (m, n), cs).astype(np.float64)
    cv = as_strided(c.reshape(-1), shape=batch + (m, n), strides=[s * c.itemsize for s in cs])
    if desc.beta != 0:
        acc = acc + float(desc.beta) * cv.astype(np.float64)
    cv[...] = acc.astype(out_dtype)


def unary(op, x, y, n, param):
    xv = x.reshape(-1)[:n].astype(np.float64)
    if op == L.SCALE:
        r = xv * np.float32(param).astype(np.float64)
    elif op == L.IDENTITY:
        r = xv
    elif op == L.RELU:
        r = np.maximum(xv, 0)
    else:
        raise NotImplementedError("unary op %d" % op)
    y.reshape(-1)[:n] = r.astype(y.dtype)


def binary(op, a, b, c, ndim, shape, a_strides, b_strides):
    """dmlhip_binary_*: NumPy broadcasting expressed as per-dimension element strides (0 = broadcast); c is dense."""
    shape = tuple(int(x) for x in shape[:ndim])
    av = _view(a, 0, shape, [int(x) for x in a_strides[:ndim]]).astype(np.float64)
    bv = _view(b, 0, shape, [int(x) for x in b_strides[:ndim]]).astype(np.float64)
    r = {L.ADD: np.add, L.SUB: np.subtract, L.MUL: np.multiply, L.DIV: np.divide, L.POW: np.power}[op](av, bv)
    n = int(np.prod(shape)) if shape else 1
    c.reshape(-1)[:n] = r.reshape(-1).astype(c.dtype)


def reduce(op, x, y, out_dtype, outer, r, inner):
    """dmlhip_reduce_*: x viewed as [outer, r, inner] -> y [outer, inner]."""
    xv = x.reshape(-1)[:outer * r * inner].astype(np.float64).reshape(outer, r, inner)
    f = {L.RSUM: np.sum, L.RMAX: np.max, L.RMIN: np.min, L.RMEAN: np.mean}[op]
    res = f(xv, axis=1) if r > 0 else np.zeros((outer, inner))
    want = np.float16 if out_dtype == L.F16 else np.float32
    if y.dtype != want:
        raise TypeError("reduce output is %s, out_dtype says %s" % (y.dtype, want))
    y.reshape(-1)[:outer * inner] = res.reshape(-1).astype(want)


def _conv_views(desc, x, w):
    import torch
    cg = desc.c // desc.group
    xt = torch.from_numpy(x.reshape(-1)[:desc.n * desc.c * desc.h * desc.w].astype(np.float64)).reshape(desc.n, desc.c, desc.h, desc.w)
    wt = torch.from_numpy(w.reshape(-1)[:desc.m * cg * desc.kh * desc.kw].astype(np.float64)).reshape(desc.m, cg, desc.kh, desc.kw)
    kw = dict(stride=(desc.stride_h, desc.stride_w), padding=(desc.pad_h, desc.pad_w), dilation=(desc.dil_h, desc.dil_w),
              groups=desc.group)
    return xt, wt, kw


def conv2d(desc, x, w, bias, y):
    """dmlhip_conv2d_*: dense NCHW / OIHW cross-correlation described by dmlhip_conv2d_desc, then the activation."""
    import torch
    xt, wt, kw = _conv_views(desc, x, w)
    bt = None if bias is None else torch.from_numpy(bias.reshape(-1)[:desc.m].astype(np.float64))
    out = _act(desc.act, torch.nn.functional.conv2d(xt, wt, bt, **kw).numpy())
    y.reshape(-1)[:out.size] = out.reshape(-1).astype(y.dtype)


def conv2d_backward(desc, which, x_or_dy, other, out):
    """dmlhip_conv2d_backward_data_f32 (dY, W -> dX) / dmlhip_conv2d_backward_weight_f32 (X, dY -> dW)."""
    import torch
    cg = desc.c // desc.group
    kw = dict(stride=(desc.stride_h, desc.stride_w), padding=(desc.pad_h, desc.pad_w), dilation=(desc.dil_h, desc.dil_w),
              groups=desc.group)
    eh, ew = (desc.kh - 1) * desc.dil_h + 1, (desc.kw - 1) * desc.dil_w + 1
    oh = (desc.h + 2 * desc.pad_h - eh) // desc.stride_h + 1
    ow = (desc.w + 2 * desc.pad_w - ew) // desc.stride_w + 1
    f64 = lambda a, shape: torch.from_numpy(a.reshape(-1)[:int(np.prod(shape))].astype(np.float64)).reshape(shape)  # noqa: E731
    if which == "data":
        dy, w = f64(x_or_dy, (desc.n, desc.m, oh, ow)), f64(other, (desc.m, cg, desc.kh, desc.kw))
        res = torch.nn.grad.conv2d_input((desc.n, desc.c, desc.h, desc.w), w, dy, **kw)
    else:
        x, dy = f64(x_or_dy, (desc.n, desc.c, desc.h, desc.w)), f64(other, (desc.n, desc.m, oh, ow))
        res = torch.nn.grad.conv2d_weight(x, (desc.m, cg, desc.kh, desc.kw), dy, **kw)
    out.reshape(-1)[:res.numel()] = res.numpy().reshape(-1).astype(out.dtype)


class Emulator:
    """Runs the calls of a HipTasklet on NumPy arrays bound to its connectors."""
    def __init__(self, workspace_bytes):
        self.workspace = np.zeros(max(int(workspace_bytes), 256), dtype=np.uint8)
        self.log = []

    def run(self, tasklet, arrays):
        """`arrays`: connector -> NumPy array (inputs are read, outputs written in place)."""
        for call in tasklet.calls:
            args = [self._arg(a, arrays) for a in call.args]
            self.log.append(call.symbol)
            if call.symbol in ("dmlhip_gemm_f16_ws", "dmlhip_gemm_f32"):
                desc, a, b, c, bias, residual, pre = args[:7]
                want = np.float16 if call.symbol.startswith("dmlhip_gemm_f16") else np.float32
                assert a.dtype == want and b.dtype == want, "%s called with %s operands" % (call.symbol, a.dtype)
                if bias is not None:
                    bias = self._typed(bias, np.float16 if desc.bias_dtype == L.F16 else np.float32)
                gemm(desc, a, b, c, bias, residual, pre)
            elif call.symbol in ("dmlhip_unary_f16", "dmlhip_unary_f32"):
                op, x, y, n, param = args[:5]
                want = np.float16 if call.symbol.endswith("f16") else np.float32
                x = self._typed(x, want)
                y = self._typed(y, want)
                unary(op, x, y, n, param)
            elif call.symbol in ("dmlhip_binary_f16", "dmlhip_binary_f32"):
                op, a, b, c, ndim, shape, sa, sb = args[:8]
                binary(op, a, b, c, ndim, shape, sa, sb)
            elif call.symbol in ("dmlhip_reduce_f16", "dmlhip_reduce_f32"):
                op, x, y, out_dtype, outer, r, inner = args[:7]
                x = self._typed(x, np.float16 if call.symbol.endswith("f16") else np.float32)
                y = self._typed(y, np.float16 if out_dtype == L.F16 else np.float32)
                reduce(op, x, y, out_dtype, outer, r, inner)
            elif call.symbol in ("dmlhip_transpose_f16", "dmlhip_transpose_f32"):
                x, y, ndim, shape, perm = args[:5]
                dt = np.float16 if call.symbol.endswith("f16") else np.float32
                x, y = self._typed(x, dt), self._typed(y, dt)
                shape, perm = tuple(shape[:ndim]), tuple(perm[:ndim])
                n = int(np.prod(shape))
                y.reshape(-1)[:n] = np.transpose(x.reshape(-1)[:n].reshape(shape), perm).reshape(-1)
            elif call.symbol in ("dmlhip_conv2d_f16", "dmlhip_conv2d_f32"):
                desc, x, w, bias, y = args[:5]
                dt = np.float16 if call.symbol.endswith("f16") else np.float32
                conv2d(desc, self._typed(x, dt), w, bias, self._typed(y, dt))
            elif call.symbol == "dmlhip_conv2d_backward_data_f32":
                desc, dy, w, dx = args[:4]
                conv2d_backward(desc, "data", dy, w, dx)
            elif call.symbol == "dmlhip_conv2d_backward_weight_f32":
                desc, x, dy, dw = args[:4]
                conv2d_backward(desc, "weight", x, dy, dw)
            elif call.symbol in ("dmlhip_softmax_backward_f16", "dmlhip_softmax_backward_f32"):
                yv, dy, dx, rows, cols = args[:5]
                y64 = yv.reshape(-1)[:rows * cols].astype(np.float64).reshape(rows, cols)
                d64 = dy.reshape(-1)[:rows * cols].astype(np.float64).reshape(rows, cols)
                p = y64 * d64
                dx.reshape(-1)[:rows * cols] = (p - y64 * p.sum(-1, keepdims=True)).reshape(-1).astype(dx.dtype)
            else:
                raise NotImplementedError("no emulation of %s" % call.symbol)

    def _typed(self, buf, dtype):
        """Workspace pointers arrive as raw bytes: view them with the element type the call implies."""
        if buf.dtype == np.uint8 and dtype != np.uint8:
            return buf[:buf.size // np.dtype(dtype).itemsize * np.dtype(dtype).itemsize].view(dtype)
        return buf

    def _arg(self, a, arrays):
        if isinstance(a, T.Ptr):
            return arrays[a.conn].reshape(-1)[a.offset:]
        if isinstance(a, T.Null):
            return None
        if isinstance(a, (T.I64, T.I32, T.USize)):
            return int(a.value)
        if isinstance(a, T.F32):
            return float(a.value)
        if isinstance(a, T.I64Array):
            return tuple(a.values)
        if isinstance(a, T.Struct):
            return a.value
        if isinstance(a, T.Workspace):
            return self.workspace[a.offset:]
        if isinstance(a, T.WorkspaceBytes):
            return self.workspace.size - a.offset
        if isinstance(a, T.Stream):
            return None
        raise NotImplementedError(type(a).__name__)


def run_state(sdfg, state, arrays):
    """Run an expanded state: `arrays` maps array names to NumPy arrays (inputs given, outputs and transients are
    allocated here when missing). Views are not supported."""
    import torch
    np_dtype = {torch.float16: np.float16, torch.float32: np.float32, torch.int64: np.int64}
    ws = max([int(getattr(n, "workspace_bytes", 0)) for n in state.library_nodes()] + [0])
    em = Emulator(ws)
    for node in state.topological_sort():
        if not getattr(node, "calls", None):
            continue
        bound = {}
        for e in list(state.in_edges(node)) + list(state.out_edges(node)):
            name = e.data.data
            d = sdfg.arrays[name]
            if d.view_of is not None:
                raise NotImplementedError("views")
            if name not in arrays:
                if name in sdfg.constants:
                    arrays[name] = sdfg.constants[name].detach().cpu().numpy().astype(np_dtype[d.dtype]).reshape(d.shape)
                else:
                    arrays[name] = np.full(d.shape, np.nan, dtype=np_dtype[d.dtype])
            bound[e.dst_conn if e.dst is node else e.src_conn] = arrays[name]
        em.run(node, bound)
    return em
