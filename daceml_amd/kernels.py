"""Tensor-level launchers: torch tensors in, one dmlhip_* call each.

PyTorch is used here only for device memory and the current HIP stream. Every function checks
device / dtype / layout, allocates the outputs (``torch.empty``, as the reference dispatcher does,
daceml/torch/dispatchers/ctypes_module.py:53-69), and calls the C ABI. There is no fallback: a
missing library or a non-zero status raises.
"""
import ctypes
from typing import Optional, Sequence

import torch

from . import _lib as L

_SUFFIX = {torch.float16: "f16", torch.float32: "f32"}
_CODE = {torch.float16: L.F16, torch.float32: L.F32}


def _stream() -> ctypes.c_void_p:
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _ptr(t: Optional[torch.Tensor]) -> ctypes.c_void_p:
    return ctypes.c_void_p(0 if t is None else t.data_ptr())


def _fn(name: str, dtype: torch.dtype):
    try:
        return getattr(L.load(), "dmlhip_%s_%s" % (name, _SUFFIX[dtype]))
    except KeyError:
        raise TypeError("dtype %s not supported by the HIP kernels (float16 / float32 only)" % dtype)


def _check(*tensors, dtype=None):
    first = None
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise ValueError("HIP kernels need device tensors; got a %s tensor" % t.device)
        if first is None:
            first = t
        elif t.device != first.device:
            raise ValueError("tensors live on different devices")
        if dtype is not None and t.dtype != dtype:
            raise TypeError("expected dtype %s, got %s" % (dtype, t.dtype))


def _dense(t: torch.Tensor) -> torch.Tensor:
    # inputs are forced contiguous, as in ctypes_module.py:58
    return t if t.is_contiguous() else t.contiguous()


_workspaces = {}


def workspace(nbytes: int, device) -> torch.Tensor:
    """Per-device scratch buffer, grown on demand and reused (kernels on one stream are ordered)."""
    key = (device.type, device.index if device.index is not None else torch.cuda.current_device())
    buf = _workspaces.get(key)
    if buf is None or buf.numel() < nbytes:
        buf = torch.empty(max(int(nbytes), 1 << 20), dtype=torch.uint8, device=device)
        _workspaces[key] = buf
    return buf


# ----------------------------------------------------------------------------- row-wise
def softmax(x: torch.Tensor, axis: int = -1, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """opset-12 Softmax: coalesce to [prod(shape[:axis]), prod(shape[axis:])]."""
    _check(x, out)
    x = _dense(x)
    axis = axis % x.dim() if x.dim() else 0
    cols = 1
    for s in x.shape[axis:]:
        cols *= s
    rows = x.numel() // cols if cols else 0
    y = torch.empty_like(x) if out is None else out
    L.check(_fn("softmax", x.dtype)(_ptr(x), _ptr(y), rows, cols, _stream()))
    return y


def softmax_backward(y: torch.Tensor, dy: torch.Tensor, axis: int = -1) -> torch.Tensor:
    _check(y, dy, dtype=y.dtype)
    y, dy = _dense(y), _dense(dy)
    axis = axis % y.dim()
    if axis != y.dim() - 1:
        raise NotImplementedError("softmax backward reduces over the single axis `axis`; only the last axis is fused")
    cols = y.shape[-1]
    rows = y.numel() // cols if cols else 0
    dx = torch.empty_like(y)
    L.check(_fn("softmax_backward", y.dtype)(_ptr(y), _ptr(dy), _ptr(dx), rows, cols, _stream()))
    return dx


def layernorm(x, gamma, beta, eps=1e-5, residual=None, want_sum=False, want_stats=False):
    """Returns (y, sum_or_None, mean_or_None, rstd_or_None); normalises over the last axis."""
    _check(x, gamma, beta, residual, dtype=x.dtype)
    x, gamma, beta = _dense(x), _dense(gamma), _dense(beta)
    if residual is not None:
        residual = _dense(residual)
        if residual.shape != x.shape:
            raise ValueError("residual must have the shape of x")
    cols = x.shape[-1]
    if gamma.numel() != cols or beta.numel() != cols:
        raise ValueError("gamma/beta must have %d elements" % cols)
    rows = x.numel() // cols if cols else 0
    y = torch.empty_like(x)
    s = torch.empty_like(x) if want_sum else None
    mean = torch.empty(rows, dtype=torch.float32, device=x.device) if want_stats else None
    rstd = torch.empty(rows, dtype=torch.float32, device=x.device) if want_stats else None
    L.check(_fn("layernorm", x.dtype)(_ptr(x), _ptr(residual), _ptr(gamma), _ptr(beta), _ptr(y), _ptr(s), _ptr(mean),
                                      _ptr(rstd), rows, cols, float(eps), _stream()))
    return y, s, mean, rstd


def layernorm_backward(dy, x, mean, rstd, gamma):
    """Returns (dx, dgamma_fp32, dbeta_fp32)."""
    _check(dy, x, gamma, dtype=x.dtype)
    _check(mean, rstd, dtype=torch.float32)
    dy, x, gamma = _dense(dy), _dense(x), _dense(gamma)
    cols = x.shape[-1]
    rows = x.numel() // cols if cols else 0
    dx = torch.empty_like(x)
    dgamma = torch.empty(cols, dtype=torch.float32, device=x.device)
    dbeta = torch.empty(cols, dtype=torch.float32, device=x.device)
    need = L.load().dmlhip_layernorm_backward_workspace_bytes(rows, cols)
    ws = workspace(need, x.device)
    L.check(_fn("layernorm_backward", x.dtype)(_ptr(dy), _ptr(x), _ptr(mean), _ptr(rstd), _ptr(gamma), _ptr(dx),
                                               _ptr(dgamma), _ptr(dbeta), rows, cols, _ptr(ws), ws.numel(), _stream()))
    return dx, dgamma, dbeta


# ----------------------------------------------------------------------------- batch normalisation
def _bn_geometry(x):
    if x.dim() < 2:
        raise ValueError("BatchNormalization needs at least [N, C], got %s" % (tuple(x.shape), ))
    n, c = x.shape[0], x.shape[1]
    hw = x.numel() // (n * c) if n * c else 0
    return n, c, hw


def batchnorm_inference(x, scale, bias, mean, var, eps=1e-5, act: int = L.ACT_NONE):
    """y = act((x - mean) / sqrt(var + eps) * scale + bias) over [N, C, ...] with given per-channel statistics."""
    _check(x, scale, bias, mean, var, dtype=x.dtype)
    x = _dense(x)
    n, c, hw = _bn_geometry(x)
    y = torch.empty_like(x)
    L.check(_fn("batchnorm_inference_act", x.dtype)(_ptr(x), _ptr(_dense(scale)), _ptr(_dense(bias)), _ptr(_dense(mean)),
                                                    _ptr(_dense(var)), _ptr(y), n, c, hw, float(eps), int(act), _stream()))
    return y


def batchnorm_training(x, scale, bias, in_mean, in_var, eps=1e-5, momentum=0.9, act: int = L.ACT_NONE):
    """Returns (y, out_mean, out_var, saved_mean, saved_var); ``momentum`` weighs the running value (ONNX); ``act`` is
    applied to the normalised value in the same kernel."""
    _check(x, scale, bias, in_mean, in_var, dtype=x.dtype)
    x = _dense(x)
    n, c, hw = _bn_geometry(x)
    y = torch.empty_like(x)
    stats = [torch.empty(c, dtype=x.dtype, device=x.device) for _ in range(4)]
    ws = workspace(L.load().dmlhip_batchnorm_workspace_bytes(n, c, hw), x.device)
    L.check(_fn("batchnorm_training_act", x.dtype)(_ptr(x), _ptr(_dense(scale)), _ptr(_dense(bias)),
                                                   _ptr(_dense(in_mean)), _ptr(_dense(in_var)), _ptr(y),
                                                   *[_ptr(t) for t in stats], n, c, hw, float(eps), float(momentum),
                                                   int(act), _ptr(ws), ws.numel(), _stream()))
    return (y, *stats)


def batchnorm_backward(dy, x, scale, saved_mean, saved_var, eps=1e-5, act: int = L.ACT_NONE, bias=None):
    """Returns (dx, dscale_fp32, dbias_fp32). With ``act`` the given gradient is the one of the activated output and
    ``bias`` is needed (the normalised value is recomputed)."""
    _check(dy, x, scale, saved_mean, saved_var, dtype=x.dtype)
    if act != L.ACT_NONE and bias is None:
        raise ValueError("batchnorm_backward with an activation needs the bias")
    dy, x = _dense(dy), _dense(x)
    n, c, hw = _bn_geometry(x)
    dx = torch.empty_like(x)
    dscale = torch.empty(c, dtype=torch.float32, device=x.device)
    dbias = torch.empty(c, dtype=torch.float32, device=x.device)
    ws = workspace(L.load().dmlhip_batchnorm_workspace_bytes(n, c, hw), x.device)
    L.check(_fn("batchnorm_backward_act", x.dtype)(_ptr(dy), _ptr(x), _ptr(_dense(scale)),
                                                   _ptr(None if bias is None else _dense(bias)), _ptr(_dense(saved_mean)),
                                                   _ptr(_dense(saved_var)), _ptr(dx), _ptr(dscale), _ptr(dbias), n, c, hw,
                                                   float(eps), int(act), _ptr(ws), ws.numel(), _stream()))
    return dx, dscale, dbias


def row_dot(a: torch.Tensor, b: torch.Tensor, keep: int) -> torch.Tensor:
    """sum(a * b) over every axis from ``keep`` on; the result has the leading ``keep`` axes."""
    _check(a, b, dtype=a.dtype)
    if a.shape != b.shape:
        raise ValueError("row_dot: operands must have one shape, got %s and %s" % (tuple(a.shape), tuple(b.shape)))
    a, b = _dense(a), _dense(b)
    rows = 1
    for d in a.shape[:keep]:
        rows *= d
    cols = a.numel() // rows if rows else 0
    y = torch.empty(tuple(a.shape[:keep]), dtype=a.dtype, device=a.device)
    L.check(_fn("row_dot", a.dtype)(_ptr(a), _ptr(b), _ptr(y), rows, cols, _stream()))
    return y


# ----------------------------------------------------------------------------- elementwise
def _bcast_strides(t: torch.Tensor, shape: Sequence[int]):
    nd = len(shape)
    pad = nd - t.dim()
    if pad < 0:
        raise ValueError("operand has more dims than the output")
    strides = []
    for i in range(nd):
        if i < pad:
            strides.append(0)
            continue
        ext, st = t.shape[i - pad], t.stride(i - pad)
        if ext == shape[i]:
            strides.append(st if ext != 1 else 0)
        elif ext == 1:
            strides.append(0)
        else:
            raise ValueError("shapes %s and %s do not broadcast" % (tuple(t.shape), tuple(shape)))
    return strides


def binary(op: int, a: torch.Tensor, b: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    _check(a, b, out, dtype=a.dtype)
    a, b = _dense(a), _dense(b)
    shape = torch.broadcast_shapes(a.shape, b.shape)
    if len(shape) > L.MAX_DIMS:
        raise NotImplementedError("more than %d dims" % L.MAX_DIMS)
    c = torch.empty(shape, dtype=a.dtype, device=a.device) if out is None else out
    sa, sb = _bcast_strides(a, shape), _bcast_strides(b, shape)
    L.check(_fn("binary", a.dtype)(op, _ptr(a), _ptr(b), _ptr(c), len(shape), L.i64_array(shape), L.i64_array(sa),
                                   L.i64_array(sb), _stream()))
    return c


def unary(op: int, x: torch.Tensor, param: float = 0.0, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    _check(x, out)
    x = _dense(x)
    y = torch.empty_like(x) if out is None else out
    L.check(_fn("unary", x.dtype)(op, _ptr(x), _ptr(y), x.numel(), float(param), _stream()))
    return y


def unary_backward(op: int, x: torch.Tensor, dy: torch.Tensor, param: float = 0.0,
                   out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``out`` may be ``dy`` itself (the gradient is then written over the one it was computed from)."""
    _check(x, dy, dtype=x.dtype)
    x, dy = _dense(x), _dense(dy)
    dx = torch.empty_like(x) if out is None else out
    if out is not None:
        _check(x, out, dtype=x.dtype)
        if not out.is_contiguous():
            raise ValueError("out must be dense")
    L.check(_fn("unary_backward", x.dtype)(op, _ptr(x), _ptr(dy), _ptr(dx), x.numel(), float(param), _stream()))
    return dx


def sum_variadic(inputs: Sequence[torch.Tensor]) -> torch.Tensor:
    if not inputs:
        raise ValueError("Sum needs at least one input")
    _check(*inputs, dtype=inputs[0].dtype)
    shape = inputs[0].shape
    for t in inputs:
        if t.shape != shape:
            raise ValueError("Sum: all inputs must have the output's shape (no broadcasting)")
    tensors = [_dense(t) for t in inputs]
    out = torch.empty_like(tensors[0])
    fn = _fn("sum", out.dtype)
    first = True
    i = 0
    while i < len(tensors):  # eight inputs per launch; later launches fold the running sum in
        chunk = tensors[i:i + (8 if first else 7)]
        ptrs = ([] if first else [out]) + chunk
        arr = (ctypes.c_void_p * len(ptrs))(*[t.data_ptr() for t in ptrs])
        L.check(fn(arr, len(ptrs), _ptr(out), out.numel(), _stream()))
        i += len(chunk)
        first = False
    return out


def bias_gelu(x: torch.Tensor, bias: Optional[torch.Tensor], want_pre: bool = False):
    _check(x, bias, dtype=x.dtype)
    x = _dense(x)
    cols = x.shape[-1]
    if bias is not None:
        bias = _dense(bias)
        if bias.numel() != cols:
            raise ValueError("bias must have %d elements" % cols)
    rows = x.numel() // cols if cols else 0
    y = torch.empty_like(x)
    pre = torch.empty_like(x) if want_pre else None
    L.check(_fn("bias_gelu", x.dtype)(_ptr(x), _ptr(bias), _ptr(y), _ptr(pre), rows, cols, _stream()))
    return y, pre


def cast(x: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    _check(x)
    x = _dense(x)
    y = torch.empty(x.shape, dtype=dtype, device=x.device)
    L.check(L.load().dmlhip_cast(_CODE[x.dtype], _CODE[dtype], _ptr(x), _ptr(y), x.numel(), _stream()))
    return y


# ----------------------------------------------------------------------------- reductions / transpose
def reduce(op: int, x: torch.Tensor, axes: Optional[Sequence[int]], keepdims: bool = True,
           out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """Reduce over `axes` (must be adjacent after normalisation; None = all)."""
    _check(x)
    x = _dense(x)
    nd = x.dim()
    axes = sorted(set(range(nd) if axes is None else [a % nd for a in axes]))
    if not axes:
        raise ValueError("empty axes")
    if axes != list(range(axes[0], axes[-1] + 1)):
        raise NotImplementedError("reduced axes must be adjacent")
    outer = 1
    for s in x.shape[:axes[0]]:
        outer *= s
    r = 1
    for a in axes:
        r *= x.shape[a]
    inner = 1
    for s in x.shape[axes[-1] + 1:]:
        inner *= s
    out_dtype = out_dtype or x.dtype
    kept = [1 if i in axes else s for i, s in enumerate(x.shape)]
    dropped = [s for i, s in enumerate(x.shape) if i not in axes]
    y = torch.empty(kept if keepdims else dropped, dtype=out_dtype, device=x.device)
    lib = L.load()
    need = lib.dmlhip_reduce_workspace_bytes(outer, r, inner)
    ws = workspace(need, x.device) if need else None
    if inner > 1 and outer > 65535:
        raise NotImplementedError("column reduction with more than 65535 outer slices")
    L.check(_fn("reduce", x.dtype)(op, _ptr(x), _ptr(y), _CODE[out_dtype], outer, r, inner, _ptr(ws),
                                   ws.numel() if ws is not None else 0, _stream()))
    return y


def transpose(x: torch.Tensor, perm: Optional[Sequence[int]] = None) -> torch.Tensor:
    _check(x)
    x = _dense(x)
    nd = x.dim()
    perm = list(reversed(range(nd))) if perm is None else [p % nd for p in perm]
    if nd > L.MAX_DIMS:
        raise NotImplementedError("more than %d dims" % L.MAX_DIMS)
    y = torch.empty([x.shape[p] for p in perm], dtype=x.dtype, device=x.device)
    L.check(_fn("transpose", x.dtype)(_ptr(x), _ptr(y), nd, L.i64_array(x.shape), L.i64_array(perm), _stream()))
    return y


def _pool_geometry(x, kernel, stride):
    if x.dim() != 4:
        raise ValueError("max_pool2d takes [N, C, H, W] tensors")
    kh, kw = kernel
    sh, sw = stride
    n, c, h, w = x.shape
    oh = (h - kh) // sh + 1 if h >= kh else 0
    ow = (w - kw) // sw + 1 if w >= kw else 0
    return n * c, h, w, kh, kw, sh, sw, oh, ow


def max_pool2d(x: torch.Tensor, kernel: Sequence[int], stride: Sequence[int]) -> torch.Tensor:
    """MaxPool without padding or dilation (floor output extents)."""
    _check(x)
    x = _dense(x)
    planes, h, w, kh, kw, sh, sw, oh, ow = _pool_geometry(x, kernel, stride)
    y = torch.empty((x.shape[0], x.shape[1], oh, ow), dtype=x.dtype, device=x.device)
    L.check(_fn("maxpool2d", x.dtype)(_ptr(x), _ptr(y), planes, h, w, kh, kw, sh, sw, _stream()))
    return y


def max_pool2d_backward(x: torch.Tensor, dy: torch.Tensor, kernel: Sequence[int], stride: Sequence[int]) -> torch.Tensor:
    _check(x, dy)
    x, dy = _dense(x), _dense(dy)
    planes, h, w, kh, kw, sh, sw, oh, ow = _pool_geometry(x, kernel, stride)
    if tuple(dy.shape) != (x.shape[0], x.shape[1], oh, ow):
        raise ValueError("gradient of shape %s for an output of shape %s" % (tuple(dy.shape), (x.shape[0], x.shape[1], oh, ow)))
    dx = torch.empty_like(x)
    L.check(_fn("maxpool2d_backward", x.dtype)(_ptr(x), _ptr(dy), _ptr(dx), planes, h, w, kh, kw, sh, sw, _stream()))
    return dx


def pad(x: torch.Tensor, pads: Sequence[int], value: float = 0.0) -> torch.Tensor:
    """ONNX Pad in constant mode: ``pads`` lists the amounts in front of every axis, then those behind (negative
    amounts crop)."""
    _check(x)
    x = _dense(x)
    nd = x.dim()
    if nd > L.MAX_DIMS:
        raise NotImplementedError("more than %d dims" % L.MAX_DIMS)
    pads = [int(p) for p in pads]
    if len(pads) != 2 * nd:
        raise ValueError("pads must hold %d amounts, got %d" % (2 * nd, len(pads)))
    begin, end = pads[:nd], pads[nd:]
    y = torch.empty([d + b + e for d, b, e in zip(x.shape, begin, end)], dtype=x.dtype, device=x.device)
    L.check(_fn("pad_constant", x.dtype)(_ptr(x), _ptr(y), nd, L.i64_array(x.shape), L.i64_array(begin), L.i64_array(end),
                                         float(value), _stream()))
    return y


# ----------------------------------------------------------------------------- contraction
def gemm(desc: "L.GemmDesc", a, b, c, bias=None, residual=None, pre_out=None):
    """Raw strided-batched GEMM; `desc` fully describes operand layout."""
    _check(a, b, c, bias, residual, pre_out)
    if a.dtype != b.dtype:
        raise TypeError("operand dtypes differ")
    L.check(_fn("gemm", a.dtype)(ctypes.byref(desc), _ptr(a), _ptr(b), _ptr(c), _ptr(bias), _ptr(residual),
                                 _ptr(pre_out), _stream()))
    return c


def _fill_desc(plan, alpha, beta, out_dtype, bias, act) -> "L.GemmDesc":
    d = L.GemmDesc()
    d.m, d.n, d.k = plan.m, plan.n, plan.k
    for i in range(3):
        d.batch[i] = plan.batch[i]
        d.a_stride_batch[i] = plan.a_stride_batch[i]
        d.b_stride_batch[i] = plan.b_stride_batch[i]
        d.c_stride_batch[i] = plan.c_stride_batch[i]
    d.a_stride_m, d.a_stride_k = plan.a_stride_m, plan.a_stride_k
    d.b_stride_k, d.b_stride_n = plan.b_stride_k, plan.b_stride_n
    d.c_stride_m = plan.c_stride_m
    d.alpha, d.beta = float(alpha), float(beta)
    d.out_dtype = _CODE[out_dtype]
    d.bias_dtype = _CODE[bias.dtype] if bias is not None else L.F16
    d.act = act
    return d


def einsum(equation: str, a: torch.Tensor, b: torch.Tensor, *, out: Optional[torch.Tensor] = None,
           out_dtype: Optional[torch.dtype] = None, alpha: float = 1.0, beta: float = 0.0,
           bias: Optional[torch.Tensor] = None, act: int = L.ACT_NONE, residual: Optional[torch.Tensor] = None,
           pre_out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Two-operand einsum as one strided batched GEMM launch.

    Operands are used with the strides they have (views are not copied). `bias` is indexed by the
    innermost output index. When one launch cannot express the equation the operands are first
    re-laid-out with the transpose kernel (still no host fallback).
    """
    from . import contraction as C
    _check(a, b, out, bias, residual, pre_out)
    if a.dtype != b.dtype:
        raise TypeError("einsum operands must share a dtype")
    out_dtype = out_dtype or a.dtype
    if a.dtype == torch.float32 and out_dtype != torch.float32:
        raise TypeError("fp32 contractions produce fp32")
    try:
        plan = C.plan_contraction(equation, a.shape, a.stride(), b.shape, b.stride())
    except C.NotApplicable:
        if bias is not None or residual is not None or pre_out is not None or out is not None or beta != 0.0:
            raise
        return _einsum_via_relayout(equation, a, b, out_dtype, alpha, act)
    if out is None:
        out = torch.empty(plan.out_shape, dtype=out_dtype, device=a.device)
    else:
        if tuple(out.shape) != tuple(plan.out_shape) or not out.is_contiguous() or out.dtype != out_dtype:
            raise ValueError("`out` must be a dense %s tensor of shape %s" % (out_dtype, plan.out_shape))
    for t in (residual, pre_out):
        if t is not None and (tuple(t.shape) != tuple(plan.out_shape) or not t.is_contiguous()
                              or t.dtype != out_dtype):
            raise ValueError("residual / pre_out must match the output's shape, dtype and layout")
    if bias is not None and (bias.dim() != 1 or bias.numel() != plan.n or not bias.is_contiguous()):
        raise ValueError("bias must be a dense vector over the innermost output index")
    x, y = (b, a) if plan.swapped else (a, b)
    desc = _fill_desc(plan, alpha, beta, out_dtype, bias, act)
    return gemm(desc, x, y, out, bias, residual, pre_out)


def _einsum_via_relayout(equation, a, b, out_dtype, alpha, act):
    from . import contraction as C
    (ta, tb), out = C.parse(equation)
    batch = [l for l in out if l in ta and l in tb]
    m_let = [l for l in out if l in ta and l not in tb]
    n_let = [l for l in out if l in tb and l not in ta]
    k_let = [l for l in ta if l in tb and l not in out]
    na = "".join(batch + m_let + k_let)
    nb = "".join(batch + k_let + n_let)
    no = "".join(batch + m_let + n_let)
    if sorted(na) != sorted(ta) or sorted(nb) != sorted(tb):
        raise C.NotApplicable("index summed inside a single operand: %s" % equation)
    a2 = transpose(a, [ta.index(l) for l in na])
    b2 = transpose(b, [tb.index(l) for l in nb])
    res = einsum("%s,%s->%s" % (na, nb, no), a2, b2, out_dtype=out_dtype, alpha=alpha, act=act)
    if no != out:
        res = transpose(res, [no.index(l) for l in out])
    return res


# ----------------------------------------------------------------------------- convolution
def _conv_desc(x_shape, w_shape, strides, pads, dilations, group, act) -> "L.Conv2dDesc":
    if len(x_shape) != 4 or len(w_shape) != 4:
        raise NotImplementedError("only 2-D convolutions (NCHW / OIHW)")
    pads = list(pads)
    if len(pads) == 4:
        if pads[0] != pads[2] or pads[1] != pads[3]:
            raise NotImplementedError("asymmetric pads")
        pads = pads[:2]
    d = L.Conv2dDesc()
    d.n, d.c, d.h, d.w = [int(v) for v in x_shape]
    d.m, d.kh, d.kw = int(w_shape[0]), int(w_shape[2]), int(w_shape[3])
    d.stride_h, d.stride_w = [int(v) for v in strides]
    d.pad_h, d.pad_w = [int(v) for v in pads]
    d.dil_h, d.dil_w = [int(v) for v in dilations]
    d.group = int(group)
    d.act = act
    if int(w_shape[1]) * d.group != d.c:
        raise ValueError("weight has %d input channels per group, expected %d" % (w_shape[1], d.c // max(d.group, 1)))
    return d


def conv_out_shape(desc: "L.Conv2dDesc"):
    oh, ow = ctypes.c_int64(), ctypes.c_int64()
    L.check(L.load().dmlhip_conv2d_out_shape(ctypes.byref(desc), ctypes.byref(oh), ctypes.byref(ow)))
    return oh.value, ow.value


def conv2d(x, w, bias=None, strides=(1, 1), pads=(0, 0), dilations=(1, 1), group=1, act: int = L.ACT_NONE):
    _check(x, w, bias, dtype=x.dtype)
    x, w = _dense(x), _dense(w)
    bias = None if bias is None else _dense(bias)
    d = _conv_desc(x.shape, w.shape, strides, pads, dilations, group, act)
    oh, ow = conv_out_shape(d)
    y = torch.empty((d.n, d.m, oh, ow), dtype=x.dtype, device=x.device)
    L.check(_fn("conv2d", x.dtype)(ctypes.byref(d), _ptr(x), _ptr(w), _ptr(bias), _ptr(y), _stream()))
    return y


def conv2d_expand_depthwise(x, w_pw, b_pw, w_dw, b_dw, stride=1, act_pw: int = L.ACT_NONE, act_dw: int = L.ACT_NONE):
    """act_dw(depthwise3x3(act_pw(conv1x1(x, w_pw) + b_pw), w_dw, stride, pad 1) + b_dw) in one kernel (fp32): the
    expanded tensor is never written to memory."""
    _check(x, w_pw, b_pw, w_dw, b_dw, dtype=torch.float32)
    x, w_pw, w_dw = _dense(x), _dense(w_pw), _dense(w_dw)
    d1 = _conv_desc(x.shape, w_pw.shape, (1, 1), (0, 0), (1, 1), 1, act_pw)
    mid = (x.shape[0], w_pw.shape[0], x.shape[2], x.shape[3])
    d2 = _conv_desc(mid, w_dw.shape, (stride, stride), (1, 1), (1, 1), w_pw.shape[0], act_dw)
    oh, ow = conv_out_shape(d2)
    y = torch.empty((d2.n, d2.m, oh, ow), dtype=x.dtype, device=x.device)
    L.check(L.load().dmlhip_conv2d_expand_depthwise_f32(ctypes.byref(d1), ctypes.byref(d2), _ptr(x), _ptr(w_pw),
                                                        _ptr(None if b_pw is None else _dense(b_pw)), _ptr(w_dw),
                                                        _ptr(None if b_dw is None else _dense(b_dw)), _ptr(y), _stream()))
    return y


def conv2d_backward(x, w, dy, strides=(1, 1), pads=(0, 0), dilations=(1, 1), group=1, need_dx=True, need_dw=True):
    """Returns (dx or None, dw or None); fp32 only."""
    _check(x, w, dy, dtype=torch.float32)
    x, w, dy = _dense(x), _dense(w), _dense(dy)
    d = _conv_desc(x.shape, w.shape, strides, pads, dilations, group, L.ACT_NONE)
    lib = L.load()
    dx = dw = None
    if need_dx:
        dx = torch.empty_like(x)
        L.check(lib.dmlhip_conv2d_backward_data_f32(ctypes.byref(d), _ptr(dy), _ptr(w), _ptr(dx), _stream()))
    if need_dw:
        dw = torch.empty_like(w)
        need = lib.dmlhip_conv2d_backward_weight_workspace_bytes(ctypes.byref(d))
        ws = workspace(need, x.device) if need else None
        L.check(lib.dmlhip_conv2d_backward_weight_f32(ctypes.byref(d), _ptr(x), _ptr(dy), _ptr(dw), _ptr(ws),
                                                      ws.numel() if ws is not None else 0, _stream()))
    return dx, dw


# ----------------------------------------------------------------------------- fused attention
def _attn_strides(t: torch.Tensor):
    if t.dim() != 4 or t.stride(3) != 1:
        raise ValueError("attention tensors are [batch0, batch1, seq, head_dim] views with a contiguous head_dim")
    return tuple(int(t.stride(i)) for i in range(3))


def _attn_desc(q, k, v, o, scale):
    d = L.AttentionDesc()
    d.batch[0], d.batch[1] = q.shape[0], q.shape[1]
    d.seq_q, d.seq_k, d.head_dim = q.shape[2], k.shape[2], q.shape[3]
    for name, t in (("q_stride", q), ("k_stride", k), ("v_stride", v), ("o_stride", o)):
        for i, sv in enumerate(_attn_strides(t)):
            getattr(d, name)[i] = sv
    d.scale = float(scale)
    return d


def _attn_mask_strides(mask, q, k):
    """Element strides over (batch0, batch1) of an additive mask broadcastable to [b0, b1, seq_q, seq_k] that does
    not depend on the query: a [.., 1, seq_k] view with contiguous keys; size-1 batch dimensions broadcast."""
    if mask.dtype != torch.float16 or mask.dim() != 4 or mask.shape[2] != 1 or mask.shape[3] != k.shape[2] or \
            (mask.shape[3] > 1 and mask.stride(3) != 1) or any(mask.shape[i] not in (1, q.shape[i]) for i in (0, 1)):
        raise ValueError("attention: the mask must be an fp16 [b0 | 1, b1 | 1, 1, seq_k] view with contiguous keys, got %s"
                         % (tuple(mask.shape), ))
    return (ctypes.c_int64 * 2)(*[0 if mask.shape[i] == 1 else int(mask.stride(i)) for i in (0, 1)])


def attention(q, k, v, scale, out=None, need_lse=True, mask=None):
    """softmax(scale * q k^T [+ mask]) v for [b0, b1, seq, 64] fp16 views (any batch / sequence strides); `mask` is
    an additive [b0 | 1, b1 | 1, 1, seq_k] fp16 tensor. Returns (out, lse)."""
    _check(q, k, v, dtype=torch.float16)
    if k.shape[:2] != q.shape[:2] or v.shape[:3] != k.shape[:3] or k.shape[3] != q.shape[3] or v.shape[3] != q.shape[3]:
        raise ValueError("attention: incompatible shapes %s %s %s" % (tuple(q.shape), tuple(k.shape), tuple(v.shape)))
    if out is None:
        out = torch.empty(q.shape, dtype=q.dtype, device=q.device)
    lse = torch.empty(q.shape[:3], dtype=torch.float32, device=q.device) if need_lse else None
    d = _attn_desc(q, k, v, out, scale)
    if mask is None:
        L.check(L.load().dmlhip_attention_f16(ctypes.byref(d), _ptr(q), _ptr(k), _ptr(v), _ptr(out), _ptr(lse), _stream()))
    else:
        _check(mask, dtype=torch.float16)
        L.check(L.load().dmlhip_attention_masked_f16(ctypes.byref(d), _ptr(q), _ptr(k), _ptr(v), _ptr(mask),
                                                     _attn_mask_strides(mask, q, k), _ptr(out), _ptr(lse), _stream()))
    return out, lse


def attention_backward(q, k, v, out, lse, dout, scale, mask=None):
    """Gradients (dq, dk, dv) of :func:`attention`; dense outputs."""
    _check(q, k, v, out, dout, dtype=torch.float16)
    dq, dk, dv = torch.empty_like(q, memory_format=torch.contiguous_format), \
        torch.empty_like(k, memory_format=torch.contiguous_format), torch.empty_like(v, memory_format=torch.contiguous_format)
    d = _attn_desc(q, k, v, out, scale)
    g = _attn_desc(dq, dk, dv, dout, scale)
    lib = L.load()
    need = lib.dmlhip_attention_backward_workspace_bytes(ctypes.byref(d))
    ws = workspace(need, q.device)
    if mask is None:
        L.check(lib.dmlhip_attention_backward_f16(ctypes.byref(d), ctypes.byref(g), _ptr(q), _ptr(k), _ptr(v), _ptr(out),
                                                  _ptr(lse), _ptr(dout), _ptr(dq), _ptr(dk), _ptr(dv), _ptr(ws), ws.numel(),
                                                  _stream()))
    else:
        _check(mask, dtype=torch.float16)
        L.check(lib.dmlhip_attention_masked_backward_f16(ctypes.byref(d), ctypes.byref(g), _ptr(q), _ptr(k), _ptr(v),
                                                         _ptr(mask), _attn_mask_strides(mask, q, k), _ptr(out), _ptr(lse),
                                                         _ptr(dout), _ptr(dq), _ptr(dk), _ptr(dv), _ptr(ws), ws.numel(),
                                                         _stream()))
    return dq, dk, dv


def reduce_sum_multi(xs: Sequence[torch.Tensor], out_dtype: Optional[torch.dtype] = None):
    """[x.sum over all axes but the last for x in xs] in one launch pair (at most eight tensors)."""
    _check(*xs, dtype=xs[0].dtype)
    xs = [_dense(x) for x in xs]
    odt = out_dtype or xs[0].dtype
    ys = [torch.empty((x.shape[-1], ), dtype=odt, device=x.device) for x in xs]
    n = len(xs)
    rows = (ctypes.c_int64 * n)(*[x.numel() // max(x.shape[-1], 1) for x in xs])
    cols = (ctypes.c_int64 * n)(*[x.shape[-1] for x in xs])
    xp = (ctypes.c_void_p * n)(*[x.data_ptr() for x in xs])
    yp = (ctypes.c_void_p * n)(*[y.data_ptr() for y in ys])
    lib = L.load()
    need = lib.dmlhip_reduce_sum_multi_workspace_bytes(n, rows, cols)
    ws = workspace(need, xs[0].device)
    L.check(_fn("reduce_sum_multi", xs[0].dtype)(n, xp, yp, L.F16 if odt == torch.float16 else L.F32, rows, cols, _ptr(ws),
                                                  ws.numel(), _stream()))
    return ys


def einsum_grouped_asum(equation: str, a_list: Sequence[torch.Tensor], b_list: Sequence[torch.Tensor], *,
                        out_dtype: Optional[torch.dtype] = None, sum_dtype: torch.dtype = torch.float32,
                        alpha: float = 1.0):
    """Like einsum_grouped (one or more pairs, no bias), and per pair the sum of the first operand over the contracted
    indices: for a weight gradient ``einsum("aij,aik->jk", dY, X)`` that is the bias gradient ``dY.sum((0, 1))``.
    Returns (outputs, sums)."""
    from . import contraction as C
    n = len(a_list)
    if n != len(b_list) or n < 1:
        raise ValueError("einsum_grouped_asum: lists differ in length")
    _check(*a_list, *b_list, dtype=None)
    a0, b0 = a_list[0], b_list[0]
    if a0.dtype != torch.float16:
        raise TypeError("einsum_grouped_asum is implemented for fp16 operands")
    for a, b in zip(a_list, b_list):
        if a.shape != a0.shape or a.stride() != a0.stride() or b.shape != b0.shape or b.stride() != b0.stride() \
                or a.dtype != a0.dtype or b.dtype != a0.dtype:
            raise ValueError("einsum_grouped_asum: every pair needs the shapes, strides and dtype of pair 0")
    out_dtype = out_dtype or a0.dtype
    plan = C.plan_contraction(equation, a0.shape, a0.stride(), b0.shape, b0.stride())
    if plan.swapped or any(e != 1 for e in plan.batch):
        raise C.NotApplicable("einsum_grouped_asum: the summed operand must be the unbatched row operand of the product")
    outs = [torch.empty(plan.out_shape, dtype=out_dtype, device=a0.device) for _ in range(n)]
    sums = [torch.empty(plan.m, dtype=sum_dtype, device=a0.device) for _ in range(n)]
    desc = _fill_desc(plan, alpha, 0.0, out_dtype, None, L.ACT_NONE)
    arr = lambda ts: (ctypes.c_void_p * n)(*[t.data_ptr() for t in ts])  # noqa: E731
    lib = L.load()
    ws = workspace(lib.dmlhip_gemm_f16_grouped_asum_workspace_bytes(ctypes.byref(desc)), a0.device)
    L.check(lib.dmlhip_gemm_f16_grouped_asum(ctypes.byref(desc), n, arr(a_list), arr(b_list), arr(outs), arr(sums),
                                             L.F32 if sum_dtype == torch.float32 else L.F16, _ptr(ws), ws.numel(),
                                             _stream()))
    return outs, sums


def einsum_sum(equation: str, a_list: Sequence[torch.Tensor], b_list: Sequence[torch.Tensor], *,
               out_dtype: Optional[torch.dtype] = None, alpha: float = 1.0, bias: Optional[torch.Tensor] = None,
               residual: Optional[torch.Tensor] = None) -> torch.Tensor:
    """alpha * sum_i einsum(equation, a_i, b_i) (+ bias) (+ residual) for fp16 operand pairs of identical shapes and
    strides (at most four), accumulated inside one launch."""
    from . import contraction as C
    n = len(a_list)
    if n != len(b_list) or n < 1:
        raise ValueError("einsum_sum: lists differ in length")
    _check(*a_list, *b_list, bias, residual, dtype=None)
    a0, b0 = a_list[0], b_list[0]
    if a0.dtype != torch.float16:
        raise TypeError("einsum_sum is implemented for fp16 operands")
    for a, b in zip(a_list, b_list):
        if a.shape != a0.shape or a.stride() != a0.stride() or b.shape != b0.shape or b.stride() != b0.stride() \
                or a.dtype != a0.dtype or b.dtype != a0.dtype:
            raise ValueError("einsum_sum: every pair needs the shapes, strides and dtype of pair 0")
    out_dtype = out_dtype or a0.dtype
    plan = C.plan_contraction(equation, a0.shape, a0.stride(), b0.shape, b0.stride())
    out = torch.empty(plan.out_shape, dtype=out_dtype, device=a0.device)
    if residual is not None and (residual.shape != out.shape or residual.dtype != out_dtype):
        raise ValueError("einsum_sum: the residual needs the output's shape and dtype")
    xs, ys = (b_list, a_list) if plan.swapped else (a_list, b_list)
    desc = _fill_desc(plan, alpha, 0.0, out_dtype, bias, L.ACT_NONE)
    arr = lambda ts: (ctypes.c_void_p * n)(*[t.data_ptr() for t in ts])  # noqa: E731
    L.check(L.load().dmlhip_gemm_f16_ksum(ctypes.byref(desc), n, arr(xs), arr(ys), _ptr(out), _ptr(bias),
                                          _ptr(_dense(residual) if residual is not None else None), _stream()))
    return out


def einsum_grouped(equation: str, a_list: Sequence[torch.Tensor], b_list: Sequence[torch.Tensor], *,
                   out_dtype: Optional[torch.dtype] = None, alpha: float = 1.0,
                   bias_list: Optional[Sequence[torch.Tensor]] = None):
    """Several fp16 two-operand einsums with the same equation, shapes and strides in one launch (at most four).
    Tensors of different groups are independent allocations; an operand may repeat (a shared input)."""
    from . import contraction as C
    n = len(a_list)
    if n != len(b_list) or (bias_list is not None and len(bias_list) != n):
        raise ValueError("einsum_grouped: lists differ in length")
    _check(*a_list, *b_list, *(bias_list or []), dtype=None)
    a0, b0 = a_list[0], b_list[0]
    if a0.dtype != torch.float16:
        raise TypeError("einsum_grouped is implemented for fp16 operands")
    for a, b in zip(a_list, b_list):
        if a.shape != a0.shape or a.stride() != a0.stride() or b.shape != b0.shape or b.stride() != b0.stride() \
                or a.dtype != a0.dtype or b.dtype != a0.dtype:
            raise ValueError("einsum_grouped: every group needs the shapes, strides and dtype of group 0")
    out_dtype = out_dtype or a0.dtype
    plan = C.plan_contraction(equation, a0.shape, a0.stride(), b0.shape, b0.stride())
    if plan.batch[0] != 1:
        raise C.NotApplicable("einsum_grouped: three batch dimensions leave no slot for the group index")
    outs = [torch.empty(plan.out_shape, dtype=out_dtype, device=a0.device) for _ in range(n)]
    xs, ys = (b_list, a_list) if plan.swapped else (a_list, b_list)
    desc = _fill_desc(plan, alpha, 0.0, out_dtype, bias_list[0] if bias_list else None, L.ACT_NONE)
    arr = lambda ts: (ctypes.c_void_p * n)(*[t.data_ptr() for t in ts])  # noqa: E731
    lib = L.load()
    need = lib.dmlhip_gemm_f16_workspace_bytes(ctypes.byref(desc))
    ws = workspace(need, a0.device)
    L.check(lib.dmlhip_gemm_f16_grouped(ctypes.byref(desc), n, arr(xs), arr(ys), arr(outs),
                                        arr(bias_list) if bias_list else None, _ptr(ws), ws.numel(), _stream()))
    return outs
