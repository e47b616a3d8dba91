"""CPU oracle: NumPy restatement of the DaCeML pure expansions on the ONNX library-node path.

TEST INFRASTRUCTURE ONLY. Nothing under ``daceml_amd/`` may import this package; it is used by
``tests/``, by ``__graft_entry__.smoke()`` and by the ``cpu_baseline`` leg of ``bench.py`` as the
checker / the timed CPU port, never as the thing shipped.

Every function cites the reference lines it restates (paths relative to the spcl/daceml tree).
Statements are kept one NumPy call per reference statement, with materialised temporaries, because
that is what ``program_for_node`` turns a pure implementation into (one map or reduction per
statement, daceml/onnx/op_implementations/utils.py:43-102) — which also makes this module the
"restated DaCe-pure CPU baseline" that bench.py times.

Pinning status (see tests/test_oracle.py):
  * every function here is pinned against an independent library routine (torch / scipy / np.einsum),
    a brute-force loop on tiny inputs, and mathematical invariants;
  * the reference holds no golden vectors for these ops (its own tests compare with NumPy/PyTorch on
    unseeded inputs), and no reference test runs them in fp16: fp16 parity is anchored on the stated
    tolerance against this fp32/fp64 oracle only ("parity unpinned" by any reference fixture).
"""
import itertools
from typing import List, Optional, Sequence, Tuple

import numpy as np
from scipy import special as _sp

# ----------------------------------------------------------------------------- elementwise


def add(A, B):
    """Add: pure_implementations.py:76-78 (``C[:] = A + B``, NumPy broadcasting)."""
    return A + B


def sub(A, B):
    """Sub: pure_implementations.py:81-83."""
    return A - B


def mul(A, B):
    """Mul: pure_implementations.py:86-88."""
    return A * B


def div(A, B):
    """Div: pure_implementations.py:91-93 (true division)."""
    return A / B


def pow_(X, Y):
    """Pow: pure_implementations.py:39-41 (``Z[:] = X ** Y``)."""
    return X**Y


def sqrt(X):
    """Sqrt: pure_implementations.py:34-36."""
    return np.sqrt(X)


def erf(x):
    """Erf: pure_implementations.py:106-108."""
    return _sp.erf(x).astype(x.dtype)


def exp(x):
    """Exp: pure_implementations.py:29-31."""
    return np.exp(x)


def log(x):
    """Log: pure_implementations.py:24-26."""
    return np.log(x)


def tanh(x):
    """Tanh: pure_implementations.py:289-291."""
    return np.tanh(x)


def relu(x):
    """Relu: pure_implementations.py:556-560 (``max(x, dtype(0))``)."""
    return np.maximum(x, x.dtype.type(0))


def reciprocal(x):
    """Reciprocal: pure_implementations.py:283-286 (``dtype(1) / x``)."""
    return x.dtype.type(1) / x


def sigmoid(x):
    """Sigmoid: pure_implementations.py:741-743 (``1 / (1 + exp(-x))`` with typed constants)."""
    one = x.dtype.type(1)
    return one / (one + np.exp(-x))


def sum_variadic(*inputs):
    """Sum: pure_implementations.py:584-646 — all inputs have the output's shape; added in order."""
    shape = inputs[0].shape
    for t in inputs:
        if t.shape != shape:
            raise ValueError("Sum: the pure expansion requires equal shapes (no broadcasting)")
    out = inputs[0].copy()
    for t in inputs[1:]:
        out = out + t
    return out


def cast(x, dtype):
    """Cast: pure_implementations.py:329-377."""
    return x.astype(dtype)


# ----------------------------------------------------------------------------- reductions


def _norm_axes(axes, ndim):
    if axes is None:
        return tuple(range(ndim))
    return tuple(a % ndim for a in axes)


def reduce_sum(data, axes=None, keepdims=1):
    """ReduceSum: pure_implementations.py:294-296; keepdims comes from the output descriptor."""
    return np.sum(data, axis=_norm_axes(axes, data.ndim), keepdims=bool(keepdims))


def reduce_max(data, axes=None, keepdims=1):
    """ReduceMax: pure_implementations.py:299-301."""
    return np.max(data, axis=_norm_axes(axes, data.ndim), keepdims=bool(keepdims))


def reduce_min(data, axes=None, keepdims=1):
    """ReduceMin: pure_implementations.py:304-306."""
    return np.min(data, axis=_norm_axes(axes, data.ndim), keepdims=bool(keepdims))


def reduce_mean(data, axes=None, keepdims=1):
    """ReduceMean: pure_implementations.py:101-103."""
    return np.mean(data, axis=_norm_axes(axes, data.ndim), keepdims=bool(keepdims))


def maxpool2d(X, kernel_shape, strides=None):
    """MaxPool "pure": img_op_implementations.py:28-161 - two spatial axes, no padding, no dilation, output extents
    rounded down; Y starts at the smallest value and takes the maximum over ``X[b, c, out*stride + h]`` (:19-21,
    :141-143)."""
    kh, kw = kernel_shape
    sh, sw = strides if strides is not None else (1, 1)
    n, c, h, w = X.shape
    oh, ow = (h - kh) // sh + 1, (w - kw) // sw + 1
    Y = np.full((n, c, oh, ow), -np.inf, dtype=X.dtype)
    for hy in range(kh):
        for hx in range(kw):
            Y = np.maximum(Y, X[:, :, hy:hy + (oh - 1) * sh + 1:sh, hx:hx + (ow - 1) * sw + 1:sw])
    return Y


def maxpool2d_backward(X, Y_grad, kernel_shape, strides):
    """DefaultMaxPoolBackward: autodiff/implementations/onnx_ops.py:284-335. Per output element the window is scanned
    row by row with a strict comparison ("deterministic argmax"), and the gradient goes to the first maximum. Windows
    that overlap add up here (as in PyTorch); the reference's tasklet assigns, which agrees wherever windows do not
    overlap - every case its own tests run."""
    kh, kw = kernel_shape
    sh, sw = strides
    n, c, oh, ow = Y_grad.shape
    X_grad = np.zeros_like(X)
    for b in range(n):
        for ch in range(c):
            for ti in range(oh):
                for tj in range(ow):
                    win = X[b, ch, sh * ti:sh * ti + kh, sw * tj:sw * tj + kw]
                    best, bi, bj = win[0, 0], 0, 0
                    for i in range(kh):
                        for j in range(kw):
                            if win[i, j] > best:
                                best, bi, bj = win[i, j], i, j
                    X_grad[b, ch, sh * ti + bi, sw * tj + bj] += Y_grad[b, ch, ti, tj]
    return X_grad


def global_average_pool(X):
    """GlobalAveragePool "pure": img_op_implementations.py:415-417; output keeps 1x1 spatial dims."""
    return np.mean(X, axis=(2, 3), keepdims=True)


# ----------------------------------------------------------------------------- softmax


def softmax(input, axis=1):
    """Softmax (opset-12 semantics): pure_implementations.py:309-319.

    Reduces over *all* axes ``range(ndim)[axis:]``; ``keepdims = (axis != 0)``.
    """
    red = tuple(range(input.ndim))[axis:]
    keepdims = axis != 0
    maximum = np.maximum.reduce(input, axis=red, keepdims=keepdims)
    exponent = np.exp(input - maximum)
    total = np.add.reduce(exponent, axis=red, keepdims=keepdims)
    return exponent / total


def softmax_backward(output, output_grad, axis):
    """DefaultSoftmaxBackward: autodiff/implementations/onnx_ops.py:237-275.

    ``prod = y*dy; sums = ReduceSum(prod, axes=[axis], keepdims=1); dx = prod - y*sums``.
    Note the backward reduces over the single axis ``axis``.
    """
    prod = mul(output, output_grad)
    sums = reduce_sum(prod, axes=[axis], keepdims=1)
    input_grad = mul(output, sums)
    return prod - input_grad


def softmax_backward_rows(output, output_grad, axis):
    """The derivative of ``softmax`` above as it is computed (opset-12: everything from ``axis`` on is one row):
    ``dx = y*dy - y * sum_{axes >= axis}(y*dy)``. DefaultSoftmaxBackward sums over the single axis ``axis``, which is this
    function when the axes behind ``axis`` have extent 1 (always the case for the last axis) and is not the derivative of
    the reference's own forward otherwise; the build's reverse node follows this function. Pinned against autograd of
    the flattened-row softmax in tests/test_oracle.py."""
    axis = axis % output.ndim
    prod = mul(output, output_grad)
    sums = reduce_sum(prod, axes=list(range(axis, output.ndim)), keepdims=1)
    return prod - mul(output, sums)


def log_softmax(input, axis=1):
    """LogSoftmax (opset-12 semantics, the axes from ``axis`` on are one row): pure_implementations.py:649-656,
    statement by statement - the logarithm is taken of the row sum."""
    red = tuple(range(input.ndim))[axis:]
    keepdims = axis != 0
    maximum = np.maximum.reduce(input, axis=red, keepdims=keepdims)
    max_sub = input - maximum
    exponent = np.exp(max_sub)
    total = np.add.reduce(exponent, axis=red, keepdims=keepdims)
    log_sum = np.log(total)
    return max_sub - log_sum


def log_softmax_backward(output, output_grad, axis):
    """DefaultLogSoftmaxBackward: autodiff/implementations/onnx_ops.py:338-373.

    ``exp_output = Exp(y); sums = ReduceSum(dy, axes=[axis], keepdims=1); dx = dy - exp_output * sums``.
    """
    exp_output = np.exp(output)
    sums = reduce_sum(output_grad, axes=[axis], keepdims=1)
    return output_grad - exp_output * sums


def attention(q, k, v, scale, mask=None):
    """The attention sub-graph as the reference expands it, node by node: Einsum(Q, K)
    (pure_implementations.py:219-252), the scalar Mul (:86-88), with ``mask`` the elementwise Add (:34-36) of a
    tensor broadcastable to the scores (a BERT encoder's padding mask is [batch, 1, 1, Sk]), Softmax(axis=-1)
    (:309-319) and Einsum(P, V). q [..., Sq, d], k [..., Sk, d], v [..., Sk, dv] with identical leading dims. Returns
    (out, lse) with lse = log(sum_j exp(scale * q.k_j + mask_j)) per query row (what a fused kernel keeps instead of
    P)."""
    lead = "abcdefgh"[:q.ndim - 2]
    scores = mul(einsum("%sik,%sjk->%sij" % (lead, lead, lead), q, k), np.asarray(scale, dtype=q.dtype))
    if mask is not None:
        scores = add(scores, mask)
    probs = softmax(scores, axis=scores.ndim - 1)
    out = einsum("%sij,%sjk->%sik" % (lead, lead, lead), probs, v)
    m = np.max(scores, axis=-1, keepdims=True)
    lse = (m + np.log(np.sum(np.exp(scores - m), axis=-1, keepdims=True)))[..., 0]
    return out, lse


def attention_backward(q, k, v, scale, out_grad, mask=None):
    """Backward of :func:`attention` as autodiff emits it: DefaultEinsumBackward for both contractions
    (autodiff/implementations/onnx_ops.py:25-138), DefaultSoftmaxBackward (:237-275), and the scalar Mul
    reversed (d/dx (x*c) = c); the Add of a constant mask passes the gradient through. Returns (dq, dk, dv)."""
    lead = "abcdefgh"[:q.ndim - 2]
    eq_s = "%sik,%sjk->%sij" % (lead, lead, lead)
    eq_o = "%sij,%sjk->%sik" % (lead, lead, lead)
    c = np.asarray(scale, dtype=q.dtype)
    scores = mul(einsum(eq_s, q, k), c)
    if mask is not None:
        scores = add(scores, mask)
    probs = softmax(scores, axis=q.ndim - 1)
    dprobs = einsum_backward(eq_o, [probs, v], out_grad, 0)
    dv = einsum_backward(eq_o, [probs, v], out_grad, 1)
    dscores = mul(softmax_backward(probs, dprobs, q.ndim - 1), c)
    dq = einsum_backward(eq_s, [q, k], dscores, 0)
    dk = einsum_backward(eq_s, [q, k], dscores, 1)
    return dq, dk, dv


# ----------------------------------------------------------------------------- LayerNorm / GELU chains


def layernorm_chain(x, gamma, beta, eps=1e-5):
    """LayerNorm as the opset-12 exporter decomposes it (no LayerNormalization node in opset 12,
    daceml/onnx/nodes/onnx_op.py:494-512): ReduceMean, Sub, Pow, ReduceMean, Add, Sqrt, Div, Mul, Add,
    each run by its pure expansion (pure_implementations.py:101-103,81-83,39-41,76-78,34-36,91-93).
    Returns (y, mean, var)."""
    two = x.dtype.type(2)
    mean = reduce_mean(x, axes=[-1], keepdims=1)
    centered = sub(x, mean)
    squared = pow_(centered, two)
    var = reduce_mean(squared, axes=[-1], keepdims=1)
    shifted = add(var, x.dtype.type(eps))
    std = sqrt(shifted)
    normed = div(centered, std)
    scaled = mul(normed, gamma)
    return add(scaled, beta), mean, var


def layernorm_backward(dy, x, gamma, eps=1e-5):
    """Gradient of layernorm_chain w.r.t. (x, gamma, beta): what reversing the nine tasklet maps with
    backward_pass_generator.py:1284-1421 and ReverseReduce (dace_nodes.py:13-105) evaluates.
    Closed form; pinned against torch.autograd in the tests."""
    n = x.shape[-1]
    mean = x.mean(axis=-1, keepdims=True)
    var = ((x - mean)**2).mean(axis=-1, keepdims=True)
    rstd = 1.0 / np.sqrt(var + x.dtype.type(eps))
    xhat = (x - mean) * rstd
    red = tuple(range(x.ndim - 1))
    dgamma = (dy * xhat).sum(axis=red)
    dbeta = dy.sum(axis=red)
    g = dy * gamma
    dx = (g - g.mean(axis=-1, keepdims=True) - xhat * (g * xhat).mean(axis=-1, keepdims=True)) * rstd
    del n
    return dx, dgamma, dbeta


def batchnorm_training(X, scale, B, in_mean, in_var, epsilon=1e-5, momentum=0.9):
    """PureBatchNormalization, training form: img_op_implementations.py:369-390, statement by statement.
    Returns (Y, out_mean, out_var, saved_mean, saved_var); the variance is the biased one and ``momentum``
    weighs the running value."""
    axis = tuple(i for i in range(X.ndim) if i != 1)
    N = 1
    for i in axis:
        N *= X.shape[i]
    bshape = [X.shape[1]] + [1] * (X.ndim - 2)
    saved_mean = np.add.reduce(X, axis=axis) / N
    X_minus_mean = X - saved_mean.reshape(bshape)
    saved_var = np.add.reduce(X_minus_mean * X_minus_mean, axis=axis) / N
    saved_var_eps = np.reshape(saved_var + epsilon, bshape)
    normalized = X_minus_mean * (1.0 / np.sqrt(saved_var_eps))
    Y = normalized * np.reshape(scale, bshape) + np.reshape(B, bshape)
    out_mean = in_mean * momentum + saved_mean * (1 - momentum)
    out_var = in_var * momentum + saved_var * (1 - momentum)
    return Y, out_mean, out_var, saved_mean, saved_var


def batchnorm_inference(X, scale, B, mean, var, epsilon=1e-5):
    """BatchNormalization with only Y connected (ONNX inference form; what tests/test_shared_input_output.py:19-43
    compares with ``F.batch_norm(X, mean, var, scale, B)``)."""
    bshape = [X.shape[1]] + [1] * (X.ndim - 2)
    return (X - np.reshape(mean, bshape)) / np.sqrt(np.reshape(var, bshape) + epsilon) * np.reshape(scale, bshape) \
        + np.reshape(B, bshape)


def batchnorm_backward(dY, X, scale, saved_mean, saved_var, epsilon=1e-5):
    """What cudnnBatchNormalizationBackwardEx returns for CuDNNBatchNormBackward
    (autodiff/implementations/onnx_ops.py:1397-1440): (dX, dscale, dB) of the training-form forward."""
    axis = tuple(i for i in range(X.ndim) if i != 1)
    N = 1
    for i in axis:
        N *= X.shape[i]
    bshape = [X.shape[1]] + [1] * (X.ndim - 2)
    invstd = 1.0 / np.sqrt(saved_var + epsilon)
    xhat = (X - saved_mean.reshape(bshape)) * invstd.reshape(bshape)
    dB = np.add.reduce(dY, axis=axis)
    dscale = np.add.reduce(dY * xhat, axis=axis)
    dX = (scale * invstd).reshape(bshape) / N * (N * dY - dB.reshape(bshape) - xhat * dscale.reshape(bshape))
    return dX, dscale, dB


def gelu_chain(x):
    """GELU as exported at opset 12: Div(x, sqrt 2), Erf, Add 1, Mul x, Mul 0.5
    (pure_implementations.py:91-93,106-108,76-78,86-88). Exact erf, not the tanh form."""
    t = x.dtype.type
    scaled = div(x, t(np.sqrt(2.0)))
    e = erf(scaled)
    shifted = add(e, t(1))
    prod = mul(x, shifted)
    return mul(prod, t(0.5))


def gelu_backward(dy, x):
    """d/dx of gelu_chain: Phi(x) + x*phi(x). Pinned against torch.autograd in the tests."""
    t = x.dtype.type
    cdf = t(0.5) * (t(1) + erf(x / t(np.sqrt(2.0))))
    pdf = np.exp(t(-0.5) * x * x) / t(np.sqrt(2.0 * np.pi))
    return dy * (cdf + x * pdf)


def swish(x):
    """Mul(x, Sigmoid(x)) — two nodes in the exported MBConv graph
    (pure_implementations.py:86-88,741-743)."""
    return mul(x, sigmoid(x))


def swish_backward(dy, x):
    s = sigmoid(x)
    return dy * (s * (1 + x * (1 - s)))


# ----------------------------------------------------------------------------- contractions


def matmul_equation(a_shape: Sequence[int], b_shape: Sequence[int]) -> str:
    """The einsum string PureMatMul lowers to: pure_implementations.py:132-191.

    Letters ``z..a`` without ``i j k``; ``pop()`` takes from the end, so the first batch letter is
    ``a``; batch dims zipped right-aligned; a dim present in one operand only gets a letter in that
    operand and the result only.
    """
    letters = [chr(ord('z') - i) for i in range(26)]
    letters = [l for l in letters if l not in ('i', 'j', 'k')]
    if len(a_shape) == 1:
        if len(b_shape) != 2:
            raise ValueError("invalid dimensions")
        return 'k,kj->j'
    if len(b_shape) == 1:
        if len(a_shape) != 2:
            raise ValueError("invalid dimensions")
        return 'ik,k->i'
    arg1, arg2, result = 'ik', 'kj', 'ij'
    for dim0, dim1 in itertools.zip_longest(reversed(a_shape[:-2]), reversed(b_shape[:-2])):
        letter = letters.pop()
        if dim0 is None:
            arg2 = letter + arg2
        elif dim1 is None:
            arg1 = letter + arg1
        else:
            arg1 = letter + arg1
            arg2 = letter + arg2
        result = letter + result
    return '{},{}->{}'.format(arg1, arg2, result)


def einsum(equation: str, *inputs):
    """PureEinsum: pure_implementations.py:219-252 — spaces stripped, ``...`` refused, then DaCe's
    ``create_einsum_sdfg`` (third-party: dace @ backport-0.13-fixes, setup.py:40), whose results the
    reference pins against ``np.einsum`` (tests/pure_expansions/test_expansions.py:387-405)."""
    equation = equation.replace(" ", "")
    if "..." in equation:
        raise NotImplementedError("PureEinsum refuses equations with an ellipsis")
    return np.einsum(equation, *inputs)


def einsum_f32_sequential(equation: str, a, b):
    """The same contraction evaluated the way the compiled pure expansion does in single precision: one fp32
    accumulator per output element, the contracted indices walked in row-major order, one rounded product and one
    rounded addition per term (the write-conflict-resolution sum of the map that ``create_einsum_sdfg`` builds for
    pure_implementations.py:219-252). It measures what fp32 summation alone costs against the fp64 value, which is
    what an fp32 kernel with some other summation order can be held to. Two operands, no repeated letters."""
    (ta, tb), to = parse_einsum(equation)
    a32, b32 = np.asarray(a, dtype=np.float32), np.asarray(b, dtype=np.float32)
    contracted = [l for l in ta if l in tb and l not in to]
    ext = {l: a32.shape[ta.index(l)] for l in contracted}
    keep_a = "".join(l for l in ta if l not in contracted)
    keep_b = "".join(l for l in tb if l not in contracted)
    step = "%s,%s->%s" % (keep_a, keep_b, to)
    out_shape = tuple((a32.shape[ta.index(l)] if l in ta else b32.shape[tb.index(l)]) for l in to)
    acc = np.zeros(out_shape, dtype=np.float32)
    for idx in np.ndindex(*[ext[l] for l in contracted]):
        pick = dict(zip(contracted, idx))
        sa = a32[tuple(pick.get(l, slice(None)) for l in ta)]
        sb = b32[tuple(pick.get(l, slice(None)) for l in tb)]
        acc += np.einsum(step, sa, sb)      # no contraction left: one fp32 product per element, then one fp32 add
    return acc


def conv2d_f32_sequential(X, W, B=None, strides=(1, 1), pads=(0, 0, 0, 0), dilations=(1, 1), group=1):
    """conv2d() in single precision in the order of PureConv2D's loop nest (img_op_implementations.py:265-288,
    314-328): the accumulator starts from the bias (or zero) and takes the products of (c, hy, hx) in that order, each
    product and each addition rounded to fp32."""
    X32, W32 = np.asarray(X, dtype=np.float32), np.asarray(W, dtype=np.float32)
    n, c, h, w = X32.shape
    m, cg, kh, kw = W32.shape
    pt, pl, pb, pr = pads
    sy, sx = strides
    dy, dx = dilations
    oh = conv_out_size(h, kh, sy, pt + pb, dy)
    ow = conv_out_size(w, kw, sx, pl + pr, dx)
    Xp = np.zeros((n, c, h + pt + pb, w + pl + pr), dtype=np.float32)
    Xp[:, :, pt:pt + h, pl:pl + w] = X32
    Y = np.zeros((n, m, oh, ow), dtype=np.float32)
    if B is not None:
        Y += np.asarray(B, dtype=np.float32).reshape(1, m, 1, 1)
    mg = m // group
    for g in range(group):
        for cc in range(cg):
            for hy in range(kh):
                for hx in range(kw):
                    patch = Xp[:, g * cg + cc, hy * dy:hy * dy + (oh - 1) * sy + 1:sy, hx * dx:hx * dx + (ow - 1) * sx + 1:sx]
                    Y[:, g * mg:(g + 1) * mg] += W32[g * mg:(g + 1) * mg, cc, hy, hx].reshape(1, mg, 1, 1) * patch[:, None]
    return Y


def matmul(A, B):
    """PureMatMul: pure_implementations.py:111-216 (refuses 1-D operands, lowers to ONNXEinsum)."""
    if A.ndim == 1 or B.ndim == 1:
        raise NotImplementedError("PureMatMul.forward_can_be_applied is False for 1-D operands")
    return einsum(matmul_equation(A.shape, B.shape), A, B)


def gemm(A, B, C=None, alpha=1.0, beta=1.0, transA=0, transB=0):
    """PureGemm: pure_implementations.py:380-553. ``Y = alpha*op(A)op(B) + beta*C``; C is indexed by
    the trailing letters of the result and its trailing dims must equal Y's (``:533-539``)."""
    arg1, arg2 = 'ik', 'kj'
    if transA == 1:
        arg1 = arg1[::-1]
    if transB == 1:
        arg2 = arg2[::-1]
    y = einsum('{},{}->ij'.format(arg1, arg2), A, B)
    if alpha != 1:
        y = y * y.dtype.type(alpha)
    if beta != 0 and C is not None:
        for c_shp, y_shp in zip(reversed(C.shape), reversed(y.shape)):
            if c_shp != y_shp:
                raise ValueError('Could not broadcast dimensions from C to Y in ONNXGemm')
        y = y + (C if beta == 1 else C * C.dtype.type(beta))
    return y


def parse_einsum(equation: str) -> Tuple[List[str], str]:
    equation = equation.replace(" ", "")
    lhs, rhs = equation.split("->")
    return lhs.split(","), rhs


def reverse_einsum_wrt_input(equation: str, input_idx: int) -> Tuple[List[int], str]:
    """reverse_einsum_wrt_input: autodiff/implementations/onnx_ops.py:25-51. Returns the indices of the
    forward inputs needed (the first operand of the new equation is the gradient of Output) and the
    equation ``out, others... -> inputs[idx]``."""
    inputs, output = parse_einsum(equation)
    exprs = [output] + inputs[:input_idx] + inputs[input_idx + 1:]
    arrays = list(range(input_idx)) + list(range(input_idx + 1, len(inputs)))
    return arrays, "{}->{}".format(",".join(exprs), inputs[input_idx])


def einsum_backward(equation: str, inputs, output_grad, wrt: int):
    """DefaultEinsumBackward: autodiff/implementations/onnx_ops.py:54-138."""
    needed, eq = reverse_einsum_wrt_input(equation, wrt)
    return einsum(eq, output_grad, *[inputs[i] for i in needed])


def transpose(data, perm=None):
    """Transpose: pure_implementations.py:322-326 (default perm = reversed axes)."""
    if perm is None:
        perm = list(reversed(range(data.ndim)))
    return np.ascontiguousarray(np.transpose(data, axes=perm))


# ----------------------------------------------------------------------------- Conv


def conv_out_size(in_size, k, stride, pad_total, dilation=1):
    """Output extent rule: shape_inference/symbolic_shape_infer.py:466-526."""
    return (in_size + pad_total - ((k - 1) * dilation + 1)) // stride + 1


def conv2d(X, W, B=None, strides=(1, 1), pads=(0, 0, 0, 0), dilations=(1, 1), group=1):
    """ONNX Conv, 2-D, NCHW/OIHW, cross-correlation.

    For stride 1 / no pad / group 1 this is PureConv2D (img_op_implementations.py:164-330):
    ``Y[b,m,oy,ox] = B[m] + sum_{c,hy,hx} W[m,c,hy,hx] * X[b,c,oy+hy,ox+hx]``, bias broadcast in the
    init state, products added onto it. Strides / symmetric pads / dilations / groups follow the
    attribute handling of CudnnConvolution (cudnn_implementations.py:148-275). ``pads`` is the ONNX
    order [top, left, bottom, right].
    """
    n, c, h, w = X.shape
    m, cg, kh, kw = W.shape
    if c != cg * group or m % group:
        raise ValueError("Conv: channel / group mismatch")
    pt, pl, pb, pr = pads
    if pt != pb or pl != pr:
        raise NotImplementedError("asymmetric pads (cudnn_implementations.py:177-181)")
    sy, sx = strides
    dy, dx = dilations
    oh = conv_out_size(h, kh, sy, pt + pb, dy)
    ow = conv_out_size(w, kw, sx, pl + pr, dx)
    Xp = np.zeros((n, c, h + pt + pb, w + pl + pr), dtype=X.dtype)
    Xp[:, :, pt:pt + h, pl:pl + w] = X
    Y = np.zeros((n, m, oh, ow), dtype=X.dtype)
    if B is not None:
        Y += B.reshape(1, m, 1, 1)
    mg = m // group
    for g in range(group):
        xs = Xp[:, g * cg:(g + 1) * cg]
        ws = W[g * mg:(g + 1) * mg]
        for hy in range(kh):
            for hx in range(kw):
                patch = xs[:, :, hy * dy:hy * dy + (oh - 1) * sy + 1:sy, hx * dx:hx * dx + (ow - 1) * sx + 1:sx]
                Y[:, g * mg:(g + 1) * mg] += np.einsum('mc,bcyx->bmyx', ws[:, :, hy, hx], patch)
    return Y


def conv2d_loops(X, W, B=None, strides=(1, 1), pads=(0, 0, 0, 0), dilations=(1, 1), group=1):
    """The same definition as seven explicit loops — the literal loop nest of
    img_op_implementations.py:265-288,314-328 extended with stride/pad/dilation/group. Tiny inputs
    only; used to pin conv2d()."""
    n, c, h, w = X.shape
    m, cg, kh, kw = W.shape
    pt, pl, pb, pr = pads
    sy, sx = strides
    dy, dx = dilations
    oh = conv_out_size(h, kh, sy, pt + pb, dy)
    ow = conv_out_size(w, kw, sx, pl + pr, dx)
    mg = m // group
    Y = np.zeros((n, m, oh, ow), dtype=np.float64)
    for b in range(n):
        for mm in range(m):
            g = mm // mg
            for oy in range(oh):
                for ox in range(ow):
                    acc = float(B[mm]) if B is not None else 0.0
                    for cc in range(cg):
                        for hy in range(kh):
                            for hx in range(kw):
                                iy = oy * sy - pt + hy * dy
                                ix = ox * sx - pl + hx * dx
                                if 0 <= iy < h and 0 <= ix < w:
                                    acc += float(W[mm, cc, hy, hx]) * float(X[b, g * cg + cc, iy, ix])
                    Y[b, mm, oy, ox] = acc
    return Y.astype(X.dtype)


def conv2d_backward(X, W, dY, strides=(1, 1), pads=(0, 0, 0, 0), dilations=(1, 1), group=1, has_bias=False):
    """dX, dW, dB of conv2d — the quantities cudnnConvolutionBackwardData/Filter/Bias return in
    autodiff/implementations/onnx_ops.py:663-703. Closed form by index reversal; pinned against
    torch.autograd in the tests."""
    n, c, h, w = X.shape
    m, cg, kh, kw = W.shape
    pt, pl, pb, pr = pads
    sy, sx = strides
    dy, dx = dilations
    oh, ow = dY.shape[2:]
    Xp = np.zeros((n, c, h + pt + pb, w + pl + pr), dtype=X.dtype)
    Xp[:, :, pt:pt + h, pl:pl + w] = X
    dXp = np.zeros_like(Xp)
    dW = np.zeros_like(W)
    mg = m // group
    for g in range(group):
        ws = W[g * mg:(g + 1) * mg]
        gy = dY[:, g * mg:(g + 1) * mg]
        for hy in range(kh):
            for hx in range(kw):
                ys = slice(hy * dy, hy * dy + (oh - 1) * sy + 1, sy)
                xs = slice(hx * dx, hx * dx + (ow - 1) * sx + 1, sx)
                patch = Xp[:, g * cg:(g + 1) * cg, ys, xs]
                dW[g * mg:(g + 1) * mg, :, hy, hx] = np.einsum('bmyx,bcyx->mc', gy, patch)
                dXp[:, g * cg:(g + 1) * cg, ys, xs] += np.einsum('bmyx,mc->bcyx', gy, ws[:, :, hy, hx])
    dX = dXp[:, :, pt:pt + h, pl:pl + w]
    dB = dY.sum(axis=(0, 2, 3)) if has_bias else None
    return np.ascontiguousarray(dX), dW, dB
