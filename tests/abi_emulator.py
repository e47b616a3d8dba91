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


def _gemm_products(desc, a, b):
    """alpha * sum_k A[b][m, k] B[b][k, n] in fp64, shape batch + (m, n)."""
    m, n, k = desc.m, desc.n, desc.k
    batch = tuple(desc.batch)
    av = _view(a, 0, batch + (m, k), tuple(desc.a_stride_batch) + (desc.a_stride_m, desc.a_stride_k))
    bv = _view(b, 0, batch + (k, n), tuple(desc.b_stride_batch) + (desc.b_stride_k, desc.b_stride_n))
    return np.matmul(av.astype(np.float64), bv.astype(np.float64)) * float(desc.alpha)


def _gemm_finish(desc, acc, c, bias, residual, pre_out):
    """The epilogue: + bias, (pre_out), activation, + residual, + beta * C, one rounding to C's type."""
    m, n = desc.m, desc.n
    batch = tuple(desc.batch)
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


def gemm(desc, a, b, c, bias, residual, pre_out):
    """dmlhip_gemm_*: C[b][m, n] = act(alpha * sum_k A[b][m, k] B[b][k, n] + bias) + residual + beta * C. `a`, `b`,
    `c`, ... are flat arrays; fp32 accumulation, one rounding to C's type."""
    _gemm_finish(desc, _gemm_products(desc, a, b), c, bias, residual, pre_out)


def _unary_value(op, xv, param):
    from scipy.special import erf
    sig = lambda v: 1 / (1 + np.exp(-v))  # noqa: E731
    return {L.ERF: lambda: erf(xv), L.SQRT: lambda: np.sqrt(xv), L.EXP: lambda: np.exp(xv), L.LOG: lambda: np.log(xv),
            L.TANH: lambda: np.tanh(xv), L.RELU: lambda: np.maximum(xv, 0), L.SIGMOID: lambda: sig(xv),
            L.RECIPROCAL: lambda: 1 / xv, L.GELU: lambda: 0.5 * xv * (1 + erf(xv / math.sqrt(2.0))),
            L.SWISH: lambda: xv * sig(xv), L.SCALE: lambda: xv * np.float32(param).astype(np.float64),
            L.IDENTITY: lambda: xv}[op]()


def _unary_derivative(op, xv, param):
    from scipy.special import erf
    sig = 1 / (1 + np.exp(-xv))
    return {L.ERF: lambda: 2 / math.sqrt(math.pi) * np.exp(-xv * xv), L.SQRT: lambda: 0.5 / np.sqrt(xv),
            L.EXP: lambda: np.exp(xv), L.LOG: lambda: 1 / xv, L.TANH: lambda: 1 - np.tanh(xv)**2,
            L.RELU: lambda: (xv > 0).astype(np.float64), L.SIGMOID: lambda: sig * (1 - sig),
            L.RECIPROCAL: lambda: -1 / (xv * xv),
            L.GELU: lambda: 0.5 * (1 + erf(xv / math.sqrt(2.0))) + xv * np.exp(-0.5 * xv * xv) / math.sqrt(2 * math.pi),
            L.SWISH: lambda: sig * (1 + xv * (1 - sig)), L.SCALE: lambda: np.full_like(xv, np.float32(param)),
            L.IDENTITY: lambda: np.ones_like(xv)}[op]()


def unary(op, x, y, n, param):
    y.reshape(-1)[:n] = _unary_value(op, x.reshape(-1)[:n].astype(np.float64), param).astype(y.dtype)


def unary_backward(op, x, dy, dx, n, param):
    """dmlhip_unary_backward_*: dx = dy * f'(x), x the forward input."""
    xv, dv = x.reshape(-1)[:n].astype(np.float64), dy.reshape(-1)[:n].astype(np.float64)
    dx.reshape(-1)[:n] = (dv * _unary_derivative(op, xv, param)).astype(dx.dtype)


def layernorm(x, residual, gamma, beta, y, sum_out, mean, rstd, rows, cols, eps):
    s = x.reshape(-1)[:rows * cols].astype(np.float64).reshape(rows, cols)
    if residual is not None:
        s = s + residual.reshape(-1)[:rows * cols].astype(np.float64).reshape(rows, cols)
        if sum_out is not None:
            sum_out.reshape(-1)[:rows * cols] = s.reshape(-1).astype(sum_out.dtype)
            s = sum_out.reshape(-1)[:rows * cols].astype(np.float64).reshape(rows, cols)   # the kernel normalises what it stores
    elif sum_out is not None:
        sum_out.reshape(-1)[:rows * cols] = s.reshape(-1).astype(sum_out.dtype)
    mu = s.mean(-1, keepdims=True)
    var = ((s - mu)**2).mean(-1, keepdims=True)
    rs = 1 / np.sqrt(var + np.float32(eps).astype(np.float64))
    out = (s - mu) * rs * gamma.reshape(-1)[:cols].astype(np.float64) + beta.reshape(-1)[:cols].astype(np.float64)
    y.reshape(-1)[:rows * cols] = out.reshape(-1).astype(y.dtype)
    if mean is not None:
        mean.reshape(-1)[:rows] = mu.reshape(-1).astype(np.float32)
    if rstd is not None:
        rstd.reshape(-1)[:rows] = rs.reshape(-1).astype(np.float32)


def layernorm_backward(dy, x, mean, rstd, gamma, dx, dgamma, dbeta, rows, cols):
    d = dy.reshape(-1)[:rows * cols].astype(np.float64).reshape(rows, cols)
    xv = x.reshape(-1)[:rows * cols].astype(np.float64).reshape(rows, cols)
    mu = mean.reshape(-1)[:rows].astype(np.float64).reshape(rows, 1)
    rs = rstd.reshape(-1)[:rows].astype(np.float64).reshape(rows, 1)
    xhat = (xv - mu) * rs
    if dgamma is not None:
        dgamma.reshape(-1)[:cols] = (d * xhat).sum(0).astype(np.float32)
    if dbeta is not None:
        dbeta.reshape(-1)[:cols] = d.sum(0).astype(np.float32)
    g = d * gamma.reshape(-1)[:cols].astype(np.float64)
    res = (g - g.mean(-1, keepdims=True) - xhat * (g * xhat).mean(-1, keepdims=True)) * rs
    dx.reshape(-1)[:rows * cols] = res.reshape(-1).astype(dx.dtype)


def _bn_tensor(buf, n, c, hw):
    return buf.reshape(-1)[:n * c * hw].astype(np.float64).reshape(n, c, hw)


def _bn_vec(buf, c):
    return buf.reshape(-1)[:c].astype(np.float64).reshape(1, c, 1)


def _act_derivative(kind, z):
    if kind == L.ACT_NONE:
        return np.ones_like(z)
    if kind == L.ACT_RELU:
        return (z > 0).astype(np.float64)
    if kind == L.ACT_SWISH:
        sg = 1 / (1 + np.exp(-z))
        return sg * (1 + z * (1 - sg))
    raise ValueError(kind)


def batchnorm_inference(x, scale, bias, mean, var, y, n, c, hw, eps, act=L.ACT_NONE):
    z = (_bn_tensor(x, n, c, hw) - _bn_vec(mean, c)) / np.sqrt(_bn_vec(var, c) + np.float32(eps).astype(np.float64)) * \
        _bn_vec(scale, c) + _bn_vec(bias, c)
    y.reshape(-1)[:n * c * hw] = _act(act, z).reshape(-1).astype(y.dtype)


def batchnorm_training(x, scale, bias, in_mean, in_var, y, out_mean, out_var, saved_mean, saved_var, n, c, hw, eps, momentum,
                       act=L.ACT_NONE):
    xv = _bn_tensor(x, n, c, hw)
    mu = xv.mean((0, 2), keepdims=True)
    var = ((xv - mu)**2).mean((0, 2), keepdims=True)
    mom = np.float32(momentum).astype(np.float64)
    new_mean = _bn_vec(in_mean, c) * mom + mu * (1 - mom)      # before the outputs are written: out_* may alias in_*
    new_var = _bn_vec(in_var, c) * mom + var * (1 - mom)
    z = (xv - mu) / np.sqrt(var + np.float32(eps).astype(np.float64)) * _bn_vec(scale, c) + _bn_vec(bias, c)
    y.reshape(-1)[:n * c * hw] = _act(act, z).reshape(-1).astype(y.dtype)
    for buf, val in ((out_mean, new_mean), (out_var, new_var), (saved_mean, mu), (saved_var, var)):
        if buf is not None:
            buf.reshape(-1)[:c] = val.reshape(-1).astype(buf.dtype)


def batchnorm_backward(dy, x, scale, bias, saved_mean, saved_var, dx, dscale, dbias, n, c, hw, eps, act=L.ACT_NONE):
    xv, d = _bn_tensor(x, n, c, hw), _bn_tensor(dy, n, c, hw)
    mu, var = _bn_vec(saved_mean, c), _bn_vec(saved_var, c)
    rs = 1 / np.sqrt(var + np.float32(eps).astype(np.float64))
    xhat = (xv - mu) * rs
    if act != L.ACT_NONE:
        d = d * _act_derivative(act, xhat * _bn_vec(scale, c) + _bn_vec(bias, c))
    if dscale is not None:
        dscale.reshape(-1)[:c] = (d * xhat).sum((0, 2)).astype(np.float32)
    if dbias is not None:
        dbias.reshape(-1)[:c] = d.sum((0, 2)).astype(np.float32)
    if dx is not None:
        g = d * _bn_vec(scale, c)
        res = (g - g.mean((0, 2), keepdims=True) - xhat * (g * xhat).mean((0, 2), keepdims=True)) * rs
        dx.reshape(-1)[:n * c * hw] = res.reshape(-1).astype(dx.dtype)


def _attn_view(desc, buf, strides, seq):
    shape = (int(desc.batch[0]), int(desc.batch[1]), int(seq), int(desc.head_dim))
    return _view(buf, 0, shape, [int(strides[0]), int(strides[1]), int(strides[2]), 1])


def _attn_probs(desc, q, k, mask, mask_stride):
    qv = _attn_view(desc, q, desc.q_stride, desc.seq_q).astype(np.float64)
    kv = _attn_view(desc, k, desc.k_stride, desc.seq_k).astype(np.float64)
    scores = np.einsum("abqd,abkd->abqk", qv, kv) * np.float32(desc.scale).astype(np.float64)
    if mask is not None:
        mv = _view(mask, 0, (int(desc.batch[0]), int(desc.batch[1]), int(desc.seq_k)),
                   [int(mask_stride[0]), int(mask_stride[1]), 1]).astype(np.float64)
        scores = scores + mv[:, :, None, :]
    m = scores.max(-1, keepdims=True)
    e = np.exp(scores - m)
    return e / e.sum(-1, keepdims=True), (m + np.log(e.sum(-1, keepdims=True)))[..., 0]


def _strided_store(buf, desc, strides, seq, value):
    shape = value.shape
    out = as_strided(buf.reshape(-1), shape=shape, strides=[int(s) * buf.itemsize for s in list(strides)[:3]] + [buf.itemsize])
    out[...] = value.astype(buf.dtype)
    del desc, seq


def attention(desc, q, k, v, o, lse, mask=None, mask_stride=None):
    """dmlhip_attention(_masked)_f16: softmax(scale q k^T [+ mask]) v on [batch0, batch1, seq, head] views."""
    p, l = _attn_probs(desc, q, k, mask, mask_stride)
    vv = _attn_view(desc, v, desc.v_stride, desc.seq_k).astype(np.float64)
    _strided_store(o, desc, desc.o_stride, desc.seq_q, np.einsum("abqk,abkd->abqd", p, vv))
    if lse is not None:
        lse.reshape(-1)[:l.size] = l.reshape(-1).astype(np.float32)


def attention_backward(desc, grad, q, k, v, o, lse, d_o, dq, dk, dv, mask=None, mask_stride=None):
    p, _ = _attn_probs(desc, q, k, mask, mask_stride)
    qv = _attn_view(desc, q, desc.q_stride, desc.seq_q).astype(np.float64)
    kv = _attn_view(desc, k, desc.k_stride, desc.seq_k).astype(np.float64)
    vv = _attn_view(desc, v, desc.v_stride, desc.seq_k).astype(np.float64)
    g = _attn_view(desc, d_o, grad.o_stride, desc.seq_q).astype(np.float64)
    dp = np.einsum("abqd,abkd->abqk", g, vv)
    ds = p * (dp - (dp * p).sum(-1, keepdims=True)) * np.float32(desc.scale).astype(np.float64)
    _strided_store(dv, desc, grad.v_stride, desc.seq_k, np.einsum("abqk,abqd->abkd", p, g))
    _strided_store(dq, desc, grad.q_stride, desc.seq_q, np.einsum("abqk,abkd->abqd", ds, kv))
    _strided_store(dk, desc, grad.k_stride, desc.seq_k, np.einsum("abqk,abqd->abkd", ds, qv))
    del o, lse


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
            elif call.symbol in ("dmlhip_unary_backward_f16", "dmlhip_unary_backward_f32"):
                op, x, dy, dx, n, param = args[:6]
                unary_backward(op, x, dy, dx, n, param)
            elif call.symbol in ("dmlhip_sum_f16", "dmlhip_sum_f32"):
                inputs, count, out, n = args[:4]
                assert len(inputs) == count
                out.reshape(-1)[:n] = sum(i.reshape(-1)[:n].astype(np.float64) for i in inputs).astype(out.dtype)
            elif call.symbol in ("dmlhip_softmax_f16", "dmlhip_softmax_f32"):
                x, y, rows, cols = args[:4]
                xv = x.reshape(-1)[:rows * cols].astype(np.float64).reshape(rows, cols)
                e = np.exp(xv - xv.max(-1, keepdims=True))
                y.reshape(-1)[:rows * cols] = (e / e.sum(-1, keepdims=True)).reshape(-1).astype(y.dtype)
            elif call.symbol in ("dmlhip_layernorm_f16", "dmlhip_layernorm_f32"):
                layernorm(*args[:11])
            elif call.symbol in ("dmlhip_layernorm_backward_f16", "dmlhip_layernorm_backward_f32"):
                a = list(args[:10])
                a[6], a[7] = self._typed(a[6], np.float32), self._typed(a[7], np.float32)   # fp32, possibly in the workspace
                layernorm_backward(*a)
            elif call.symbol == "dmlhip_layernorm_backward_grads_f16":
                kinds = {L.F16: np.float16, L.F32: np.float32}
                a = list(args[:8]) + list(args[9:11])
                f32 = [np.zeros(args[10], np.float32), np.zeros(args[10], np.float32)]
                typed = [self._typed(a[6], kinds[args[8]]), self._typed(a[7], kinds[args[8]])]
                a[6], a[7] = f32
                layernorm_backward(*a)
                for dst, src in zip(typed, f32):   # fp32 column sums, rounded once
                    dst.reshape(-1)[:args[10]] = src.astype(kinds[args[8]])
            elif call.symbol == "dmlhip_cast":
                kinds = {L.F16: np.float16, L.F32: np.float32}
                src, dst, n = self._typed(args[2], kinds[args[0]]), self._typed(args[3], kinds[args[1]]), args[4]
                dst.reshape(-1)[:n] = src.reshape(-1)[:n].astype(kinds[args[1]])
            elif call.symbol == "dmlhip_attention_f16":
                attention(*args[:6])
            elif call.symbol == "dmlhip_attention_masked_f16":
                desc, q, k, v, mask, ms, o, lse = args[:8]
                attention(desc, q, k, v, o, lse, mask, ms)
            elif call.symbol == "dmlhip_attention_backward_f16":
                attention_backward(*args[:11])
            elif call.symbol == "dmlhip_attention_masked_backward_f16":
                desc, grad, q, k, v, mask, ms, o, lse, d_o, dq, dk, dv = args[:13]
                attention_backward(desc, grad, q, k, v, o, lse, d_o, dq, dk, dv, mask, ms)
            elif call.symbol == "dmlhip_gemm_f16_grouped":
                desc, groups, a, b, c, bias = args[:6]
                for i in range(groups):
                    bi = None if bias is None else self._typed(bias[i], np.float16 if desc.bias_dtype == L.F16 else np.float32)
                    gemm(desc, a[i], b[i], c[i], bi, None, None)
            elif call.symbol == "dmlhip_gemm_f16_grouped_asum":
                desc, groups, a, b, c, asum, asum_dtype = args[:7]
                for i in range(groups):
                    gemm(desc, a[i], b[i], c[i], None, None, None)
                    av = _view(a[i], 0, (desc.m, desc.k), (desc.a_stride_m, desc.a_stride_k)).astype(np.float64)
                    asum[i].reshape(-1)[:desc.m] = av.sum(1).astype(np.float16 if asum_dtype == L.F16 else np.float32)
            elif call.symbol == "dmlhip_gemm_f16_ksum":
                desc, groups, a, b, c, bias, residual = args[:7]
                # the kernel keeps the sum of the products in its accumulators: one rounding at the end
                total = sum(_gemm_products(desc, a[i], b[i]) for i in range(groups))
                if bias is not None:
                    bias = self._typed(bias, np.float16 if desc.bias_dtype == L.F16 else np.float32)
                _gemm_finish(desc, total, c, bias, residual, None)
            elif call.symbol in ("dmlhip_binary_f16", "dmlhip_binary_f32"):
                op, a, b, c, ndim, shape, sa, sb = args[:8]
                dt = np.float16 if call.symbol.endswith("f16") else np.float32
                binary(op, self._typed(a, dt), self._typed(b, dt), self._typed(c, dt), ndim, shape, sa, sb)
            elif call.symbol in ("dmlhip_reduce_f16", "dmlhip_reduce_f32"):
                op, x, y, out_dtype, outer, r, inner = args[:7]
                x = self._typed(x, np.float16 if call.symbol.endswith("f16") else np.float32)
                y = self._typed(y, np.float16 if out_dtype == L.F16 else np.float32)
                reduce(op, x, y, out_dtype, outer, r, inner)
            elif call.symbol in ("dmlhip_reduce_sum_multi_f16", "dmlhip_reduce_sum_multi_f32"):
                count, xs, ys, out_dtype, rows, cols = args[:6]
                assert len(xs) == len(ys) == count <= L.MULTI_MAX if hasattr(L, "MULTI_MAX") else len(xs) == len(ys) == count
                want = np.float16 if out_dtype == L.F16 else np.float32
                for x, y, r, c in zip(xs, ys, rows[:count], cols[:count]):
                    if y.dtype != want:
                        raise TypeError("multi reduce output is %s, out_dtype says %s" % (y.dtype, want))
                    y.reshape(-1)[:c] = x.reshape(-1)[:r * c].astype(np.float64).reshape(r, c).sum(0).astype(want)
            elif call.symbol in ("dmlhip_transpose_f16", "dmlhip_transpose_f32"):
                x, y, ndim, shape, perm = args[:5]
                dt = np.float16 if call.symbol.endswith("f16") else np.float32
                x, y = self._typed(x, dt), self._typed(y, dt)
                shape, perm = tuple(shape[:ndim]), tuple(perm[:ndim])
                n = int(np.prod(shape))
                y.reshape(-1)[:n] = np.transpose(x.reshape(-1)[:n].reshape(shape), perm).reshape(-1)
            elif call.symbol in ("dmlhip_maxpool2d_f16", "dmlhip_maxpool2d_f32", "dmlhip_maxpool2d_backward_f16",
                                 "dmlhip_maxpool2d_backward_f32"):
                import torch
                backward = "backward" in call.symbol
                x, a1 = args[0], args[1]
                planes, h, w, kh, kw, sh, sw = args[3:10] if backward else args[2:9]
                xt = torch.from_numpy(x.reshape(-1)[:planes * h * w].astype(np.float64).reshape(1, planes, h, w))
                oh, ow = ((h - kh) // sh + 1 if h >= kh else 0), ((w - kw) // sw + 1 if w >= kw else 0)
                if not backward:
                    out = torch.nn.functional.max_pool2d(xt, (kh, kw), (sh, sw)).numpy()
                    a1.reshape(-1)[:out.size] = out.reshape(-1).astype(a1.dtype)
                else:
                    dx = args[2]
                    xt.requires_grad_(True)
                    g = torch.from_numpy(a1.reshape(-1)[:planes * oh * ow].astype(np.float64).reshape(1, planes, oh, ow))
                    torch.nn.functional.max_pool2d(xt, (kh, kw), (sh, sw)).backward(g)
                    dx.reshape(-1)[:planes * h * w] = xt.grad.numpy().reshape(-1).astype(dx.dtype)
            elif call.symbol in ("dmlhip_pad_constant_f16", "dmlhip_pad_constant_f32"):
                x, y, ndim, shape, begin, end, value = args[:7]
                dt = np.float16 if call.symbol.endswith("f16") else np.float32
                x, y = self._typed(x, dt), self._typed(y, dt)
                shape, begin, end = (tuple(int(v) for v in t[:ndim]) for t in (shape, begin, end))
                src = x.reshape(-1)[:int(np.prod(shape))].reshape(shape)
                # negative amounts crop first, positive ones pad afterwards
                src = src[tuple(slice(max(-b, 0), d - max(-e, 0)) for d, b, e in zip(shape, begin, end))]
                out = np.pad(src, [(max(b, 0), max(e, 0)) for b, e in zip(begin, end)], constant_values=dt(value))
                y.reshape(-1)[:out.size] = out.reshape(-1)
            elif call.symbol in ("dmlhip_conv2d_f16", "dmlhip_conv2d_f32"):
                desc, x, w, bias, y = args[:5]
                dt = np.float16 if call.symbol.endswith("f16") else np.float32
                conv2d(desc, self._typed(x, dt), w, bias, self._typed(y, dt))
            elif call.symbol.startswith("dmlhip_batchnorm_inference"):
                x, scale, bias, mean, var, y, n, c, hw, eps = args[:10]
                batchnorm_inference(x, scale, bias, mean, var, y, n, c, hw, eps, args[10] if "_act_" in call.symbol else L.ACT_NONE)
            elif call.symbol.startswith("dmlhip_batchnorm_training"):
                batchnorm_training(*args[:15], args[15] if "_act_" in call.symbol else L.ACT_NONE)
            elif call.symbol.startswith("dmlhip_batchnorm_backward"):
                if "_act_" in call.symbol:
                    dy, x, scale, bias, sm, sv, dx, ds, db, n, c, hw, eps, act = args[:14]
                else:
                    dy, x, scale, sm, sv, dx, ds, db, n, c, hw, eps = args[:12]
                    bias, act = None, L.ACT_NONE
                batchnorm_backward(dy, x, scale, bias, sm, sv, dx, self._typed(ds, np.float32) if ds is not None else None,
                                   self._typed(db, np.float32) if db is not None else None, n, c, hw, eps, act)
            elif call.symbol == "dmlhip_conv2d_gated_f32":
                desc, x, gate, w, bias, y = args[:6]
                n = desc.n * desc.c * desc.h * desc.w
                gated = (x.reshape(-1)[:n].astype(np.float64).reshape(desc.n, desc.c, desc.h * desc.w) *
                         gate.reshape(-1)[:desc.n * desc.c].astype(np.float64).reshape(desc.n, desc.c, 1))
                conv2d(desc, gated.reshape(-1), w, bias, y)
            elif call.symbol == "dmlhip_conv2d_expand_depthwise_f32":
                pw, dw, x, w_pw, b_pw, w_dw, b_dw, y = args[:8]
                mid = np.empty(pw.n * pw.m * pw.h * pw.w, dtype=np.float64)   # the expanded tensor is never rounded to memory
                conv2d(pw, x, w_pw, b_pw, mid)
                conv2d(dw, mid, w_dw, b_dw, y)
            elif call.symbol in ("dmlhip_row_dot_f16", "dmlhip_row_dot_f32"):
                a, b, y, rows, cols = args[:5]
                av = a.reshape(-1)[:rows * cols].astype(np.float64).reshape(rows, cols)
                bv = b.reshape(-1)[:rows * cols].astype(np.float64).reshape(rows, cols)
                y.reshape(-1)[:rows] = (av * bv).sum(1).astype(y.dtype)
            elif call.symbol in ("dmlhip_row_affine_f16", "dmlhip_row_affine_f32"):
                a, sc, t, scale, y, rows, cols = args[:7]
                av = a.reshape(-1)[:rows * cols].astype(np.float64).reshape(rows, cols)
                f = 1.0 if scale is None else float(scale.reshape(-1)[0])
                res = av * sc.reshape(-1)[:rows].astype(np.float64).reshape(rows, 1) + \
                    t.reshape(-1)[:rows].astype(np.float64).reshape(rows, 1) * f
                y.reshape(-1)[:rows * cols] = res.reshape(-1).astype(y.dtype)
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
        if isinstance(a, T.PtrArray):
            return [arrays[c].reshape(-1) for c in a.conns]
        if isinstance(a, T.Struct):
            return a.value
        if isinstance(a, T.Workspace):
            return self.workspace[a.offset:]
        if isinstance(a, T.WorkspaceBytes):
            return self.workspace.size - a.offset
        if isinstance(a, T.Stream):
            return None
        raise NotImplementedError(type(a).__name__)


def _memory(sdfg, arrays, name, np_dtype):
    """The flat memory an array name stands for: its own allocation, or for a view the base's memory from the view's
    offset on (descriptors carry the view's strides)."""
    d = sdfg.arrays[name]
    if d.view_of is not None:
        return _memory(sdfg, arrays, d.view_of, np_dtype).reshape(-1)[d.view_offset:]
    if name not in arrays:
        if name in sdfg.constants:
            arrays[name] = sdfg.constants[name].detach().cpu().numpy().astype(np_dtype[d.dtype]).reshape(d.shape)
        else:
            arrays[name] = np.full(d.shape, np.nan, dtype=np_dtype[d.dtype])
    return arrays[name]


def run_state(sdfg, state, arrays):
    """Run an expanded state: `arrays` maps array names to NumPy arrays (inputs given, outputs and transients are
    allocated here when missing)."""
    import torch
    np_dtype = {torch.float16: np.float16, torch.float32: np.float32, torch.int64: np.int64}
    ws = max([int(getattr(n, "workspace_bytes", 0)) for n in state.nodes()] + [0])
    em = Emulator(ws)
    for node in state.topological_sort():
        if not getattr(node, "calls", None):
            continue
        bound = {}
        for e in list(state.in_edges(node)) + list(state.out_edges(node)):
            bound[e.dst_conn if e.dst is node else e.src_conn] = _memory(sdfg, arrays, e.data.data, np_dtype)
        em.run(node, bound)
    return em


def run_sdfg(sdfg, arrays):
    """Every state in order (forward, then backward). Returns the list of calls made."""
    log = []
    for st in sdfg.states():
        log += run_state(sdfg, st, arrays).log
    return log


def run_sdfg_in_arena(sdfg, arrays):
    """The whole SDFG as ``CompiledSDFG(reuse_transients=True)`` runs it: the nodes in the order
    ``memory_plan.launch_order`` chooses, the transients as pieces of one arena at the offsets
    ``memory_plan.place_transients`` gives them. The arena starts out as NaN bit patterns, so a transient read before it
    is written, or after another one took over its bytes, shows in the results. Returns (order of node labels, plan,
    arena bytes)."""
    import torch
    from daceml_amd import memory_plan
    np_dtype = {torch.float16: np.float16, torch.float32: np.float32, torch.int64: np.int64}
    order = memory_plan.launch_order(sdfg, small_peak=True)
    plan = memory_plan.place_transients(sdfg, order)
    total = max([off + memory_plan.nbytes(sdfg.arrays[n]) for n, off in plan.items()] + [0])
    arena = np.full(total, 0xFF, dtype=np.uint8)
    for name, off in plan.items():
        d = sdfg.arrays[name]
        arrays[name] = arena[off:off + memory_plan.nbytes(d)].view(np_dtype[d.dtype]).reshape(d.shape)
    ws = max([int(getattr(n, "workspace_bytes", 0)) for _, n in order] + [0])
    em = Emulator(ws)
    for state, node in order:
        if not getattr(node, "calls", None):
            continue
        bound = {}
        for e in list(state.in_edges(node)) + list(state.out_edges(node)):
            bound[e.dst_conn if e.dst is node else e.src_conn] = _memory(sdfg, arrays, e.data.data, np_dtype)
        em.run(node, bound)
    return [n.label for _, n in order], plan, total


def run_program(program, arrays):
    """Run a lowered TaskletProgram (daceml_amd/lowering.py): `arrays` maps the program's array names to NumPy arrays
    (arguments given; transients, constants and missing outputs are allocated here). Connectors address their array
    from the element offset the lowering recorded for them."""
    import torch
    np_dtype = {torch.float16: np.float16, torch.float32: np.float32, torch.int64: np.int64}
    for name, d in program.arrays.items():
        if name not in arrays:
            if name in program.constants:
                arrays[name] = program.constants[name].detach().cpu().numpy().astype(np_dtype[d.dtype]).reshape(d.shape)
            else:
                arrays[name] = np.full(d.shape, np.nan, dtype=np_dtype[d.dtype])
    em = Emulator(program.workspace_bytes)
    for spec in program.tasklets:
        bound = {}
        for conn, arr in list(spec.inputs.items()) + list(spec.outputs.items()):
            bound[conn] = arrays[arr].reshape(-1)[spec.offsets.get(conn, 0):]
        em.run(spec, bound)
    return em
