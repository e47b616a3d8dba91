"""The "hip" implementations of the ONNX library nodes: each ``forward`` returns a ``HipTasklet`` that
calls one (or a few) hand-written gfx950 kernels through the ``dmlhip_*`` C ABI.

Counterparts in the reference: the "pure" expansions of
daceml/onnx/op_implementations/pure_implementations.py and img_op_implementations.py (whose results
these must reproduce) and the cuDNN expansion of cudnn_implementations.py (whose role — a native
library behind an expansion — these play). ``forward_can_be_applied`` never raises: anything outside
what the kernels cover returns False.
"""
import math
from typing import List, Optional, Sequence, Tuple

import torch

from ... import _lib as L
from ... import contraction as C
from ...hip_tasklet import (F32, I32, I64, HipCall, HipTasklet, I64Array, Null, Ptr, PtrArray, Stream, Struct,
                            USize, ViewTasklet, Workspace, WorkspaceBytes)
from ...sdfg import (FLOAT_DTYPES, SDFG, AccessNode, Array, SDFGState, in_desc_with_name, out_desc_with_name)
from ..forward_implementation_abc import ONNXForward
from ..nodes import ONNXOp
from .utils import op_implementation

IMPL = "hip"
_SFX = {torch.float16: "f16", torch.float32: "f32"}
_CODE = {torch.float16: L.F16, torch.float32: L.F32}
_ITEMSIZE = {torch.float16: 2, torch.float32: 4}
_ACT = {"none": L.ACT_NONE, "gelu": L.ACT_GELU, "swish": L.ACT_SWISH, "sigmoid": L.ACT_SIGMOID, "relu": L.ACT_RELU}


# ----------------------------------------------------------------------------- helpers
def _connected(node: ONNXOp, state: SDFGState, is_input: bool) -> List[str]:
    edges = state.in_edges(node) if is_input else state.out_edges(node)
    return [e.dst_conn if is_input else e.src_conn for e in edges]


def _has_in(node, state, name) -> bool:
    return name in _connected(node, state, True)


def _has_out(node, state, name) -> bool:
    return name in _connected(node, state, False)


def _descs(node, state, sdfg):
    ins = {e.dst_conn: sdfg.arrays[e.data.data] for e in state.in_edges(node)}
    outs = {e.src_conn: sdfg.arrays[e.data.data] for e in state.out_edges(node)}
    return ins, outs


def _float_ok(*descs: Array) -> bool:
    if not descs:
        return False
    dt = descs[0].dtype
    return dt in FLOAT_DTYPES and all(d.dtype == dt for d in descs)


def _dense(*descs: Array) -> bool:
    return all(d.is_contiguous() for d in descs)


def _prod(xs: Sequence[int]) -> int:
    n = 1
    for x in xs:
        n *= int(x)
    return n


def _tasklet(node, state, calls, workspace_bytes=0, flops=0, bytes_moved=0, kind=""):
    return HipTasklet(node.label + "_hip", _connected(node, state, True), _connected(node, state, False), calls,
                      workspace_bytes, flops, bytes_moved, kind or node.schema.name)


def _opt(node, state, name, is_input=True):
    present = _has_in(node, state, name) if is_input else _has_out(node, state, name)
    return Ptr(name) if present else Null()


def _nbytes(*descs: Array) -> int:
    return sum(d.total_size * (2 if d.dtype == torch.float16 else 4) for d in descs)


# ----------------------------------------------------------------------------- contractions
def _gemm_struct(plan: C.GemmPlan, alpha, beta, out_dtype, bias_dtype, act) -> L.GemmDesc:
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
    d.bias_dtype = _CODE[bias_dtype]
    d.act = act
    d.bias_along_m = 0
    return d


def _einsum_plan(equation: str, a: Array, b: Array) -> Optional[C.GemmPlan]:
    try:
        return C.plan_contraction(equation, a.shape, a.strides, b.shape, b.strides)
    except (C.NotApplicable, ValueError):
        return None


def _einsum_can_apply(equation: str, inputs: List[Array], out: Array, allow_f32_out=False) -> bool:
    if "..." in equation or not inputs or not _float_ok(*inputs):
        return False
    if out.dtype != inputs[0].dtype and not (allow_f32_out and out.dtype == torch.float32):
        return False
    if not out.is_contiguous():
        return False
    try:
        if len(inputs) == 1:
            perm = C.transpose_perm(equation)
            return perm is not None and inputs[0].is_contiguous() and len(perm) <= L.MAX_DIMS
        if len(inputs) != 2:
            return False
        plan = _einsum_plan(equation, inputs[0], inputs[1])
        return plan is not None and tuple(plan.out_shape) == tuple(out.shape)
    except (C.NotApplicable, ValueError):
        return False


def _einsum_tasklet(node, state, equation, a_conn, b_conn, out_conn, a: Array, b: Array, out: Array, alpha=1.0,
                    beta=0.0, act=L.ACT_NONE, bias: Optional[str] = None, bias_desc: Optional[Array] = None,
                    residual: Optional[str] = None, pre_out: Optional[str] = None):
    plan = C.plan_contraction(equation, a.shape, a.strides, b.shape, b.strides)
    desc = _gemm_struct(plan, alpha, beta, out.dtype, bias_desc.dtype if bias_desc is not None else out.dtype, act)
    x, y = (b_conn, a_conn) if plan.swapped else (a_conn, b_conn)
    ptrs = [Struct(desc, "dmlhip_gemm_desc"), Ptr(x), Ptr(y), Ptr(out_conn), Ptr(bias) if bias else Null(),
            Ptr(residual) if residual else Null(), Ptr(pre_out) if pre_out else Null()]
    ws = 0
    if a.dtype == torch.float16:
        import ctypes
        ws = L.load().dmlhip_gemm_f16_workspace_bytes(ctypes.byref(desc))
        call = HipCall("dmlhip_gemm_f16_ws", ptrs + [Workspace(), WorkspaceBytes(), Stream()])
    else:
        call = HipCall("dmlhip_gemm_f32", ptrs + [Stream()])
    extra = [d for d in (bias_desc, ) if d is not None]
    return _tasklet(node, state, [call], workspace_bytes=ws, flops=plan.flops, bytes_moved=_nbytes(a, b, out, *extra),
                    kind="gemm")


@op_implementation(op="Einsum", name=IMPL)
class HipEinsum(ONNXForward):
    """PureEinsum (pure_implementations.py:219-252): two-operand contractions become one MFMA GEMM
    launch; one-operand permutations become the transpose kernel (EinsumTranspose, :746-778)."""
    @staticmethod
    def forward_can_be_applied(node, state, sdfg) -> bool:
        try:
            ins = [sdfg.arrays[e.data.data] for e in node.iter_inputs_in_onnx_order(state)]
            out = out_desc_with_name(node, state, sdfg, "Output")
            return _einsum_can_apply(node.equation.replace(" ", ""), ins, out)
        except Exception:
            return False

    @staticmethod
    def forward(node, state, sdfg):
        eq = node.equation.replace(" ", "")
        edges = node.iter_inputs_in_onnx_order(state)
        ins = [sdfg.arrays[e.data.data] for e in edges]
        out = out_desc_with_name(node, state, sdfg, "Output")
        if len(ins) == 1:
            perm = C.transpose_perm(eq)
            call = HipCall("dmlhip_transpose_" + _SFX[out.dtype],
                           [Ptr("Inputs__0"), Ptr("Output"), I32(len(perm)), I64Array(tuple(ins[0].shape)),
                            I64Array(tuple(perm)), Stream()])
            return _tasklet(node, state, [call], bytes_moved=_nbytes(ins[0], out), kind="transpose")
        return _einsum_tasklet(node, state, eq, "Inputs__0", "Inputs__1", "Output", ins[0], ins[1], out)


def _input_sum_ok(plan, a: Array, s: Array) -> bool:
    """The row-sum result of the contraction kernel: the summed operand is the unbatched row operand A, stored as a
    dense [k, m] matrix; the sums are a dense vector of m fp16 / fp32 values."""
    return (plan is not None and not plan.swapped and all(e == 1 for e in plan.batch) and a.dtype == torch.float16
            and a.is_contiguous() and a.shape[-1] == plan.m and a.total_size == plan.m * plan.k
            and s.dtype in FLOAT_DTYPES and s.is_contiguous() and s.total_size == plan.m)


def _asum_tasklet(node, state, eq, alpha, a, b, out, sum_desc, a_conns, b_conns, out_conns, sum_conns):
    import ctypes
    n = len(a)
    plan = C.plan_contraction(eq, a[0].shape, a[0].strides, b[0].shape, b[0].strides)
    desc = _gemm_struct(plan, alpha, 0.0, out[0].dtype, out[0].dtype, L.ACT_NONE)
    ws = L.load().dmlhip_gemm_f16_grouped_asum_workspace_bytes(ctypes.byref(desc))
    call = HipCall("dmlhip_gemm_f16_grouped_asum",
                   [Struct(desc, "dmlhip_gemm_desc"), I32(n), PtrArray(tuple(a_conns)), PtrArray(tuple(b_conns)),
                    PtrArray(tuple(out_conns)), PtrArray(tuple(sum_conns)), I32(_CODE[sum_desc.dtype]), Workspace(),
                    WorkspaceBytes(), Stream()])
    return _tasklet(node, state, [call], workspace_bytes=ws, flops=plan.flops * n,
                    bytes_moved=sum(_nbytes(a[i], b[i], out[i]) for i in range(n)), kind="gemm")


@op_implementation(op="FusedEinsum", name=IMPL)
class HipFusedEinsum(ONNXForward):
    """A contraction with the scale / bias Add / activation / residual Add that followed it in the
    exported graph folded into the GEMM epilogue, and Transposes of its operands folded into operand
    strides (the job of transformation/einsum_fusion.py:102-151 in the reference)."""
    @staticmethod
    def forward_can_be_applied(node, state, sdfg) -> bool:
        try:
            ins, outs = _descs(node, state, sdfg)
            if "Inputs__0" not in ins or "Inputs__1" not in ins or "Inputs__2" in ins:
                return False
            out = outs["Output"]
            if node.activation not in _ACT:
                return False
            if not _einsum_can_apply(node.equation.replace(" ", ""), [ins["Inputs__0"], ins["Inputs__1"]], out,
                                     allow_f32_out=True):
                return False
            plan = _einsum_plan(node.equation.replace(" ", ""), ins["Inputs__0"], ins["Inputs__1"])
            if "Bias" in ins:
                b = ins["Bias"]
                if not (b.dtype in FLOAT_DTYPES and b.is_contiguous() and b.total_size == plan.n
                        and b.shape[-1] == plan.n):
                    return False
            for name, d in (("Residual", ins.get("Residual")), ("PreActivation", outs.get("PreActivation"))):
                if d is not None and not (d.is_contiguous() and tuple(d.shape) == tuple(out.shape)
                                          and d.dtype == out.dtype):
                    return False
            if "InputSum" in outs:
                plain = set(ins) == {"Inputs__0", "Inputs__1"} and set(outs) == {"Output", "InputSum"}
                if not (plain and node.activation == "none" and not node.accumulate
                        and _input_sum_ok(plan, ins["Inputs__0"], outs["InputSum"])):
                    return False
            return True
        except Exception:
            return False

    @staticmethod
    def forward(node, state, sdfg):
        ins, outs = _descs(node, state, sdfg)
        if "InputSum" in outs:
            return _asum_tasklet(node, state, node.equation.replace(" ", ""), node.alpha, [ins["Inputs__0"]],
                                 [ins["Inputs__1"]], [outs["Output"]], outs["InputSum"], ["Inputs__0"], ["Inputs__1"],
                                 ["Output"], ["InputSum"])
        return _einsum_tasklet(node, state, node.equation.replace(" ", ""), "Inputs__0", "Inputs__1", "Output",
                               ins["Inputs__0"], ins["Inputs__1"], outs["Output"], alpha=node.alpha,
                               beta=1.0 if node.accumulate else 0.0, act=_ACT[node.activation],
                               bias="Bias" if "Bias" in ins else None, bias_desc=ins.get("Bias"),
                               residual="Residual" if "Residual" in ins else None,
                               pre_out="PreActivation" if "PreActivation" in outs else None)


@op_implementation(op="MatMul", name=IMPL)
class HipMatMul(ONNXForward):
    """PureMatMul (pure_implementations.py:111-216): same einsum lowering, then one GEMM launch."""
    @staticmethod
    def forward_can_be_applied(node, state, sdfg) -> bool:
        try:
            a = in_desc_with_name(node, state, sdfg, "A")
            b = in_desc_with_name(node, state, sdfg, "B")
            y = out_desc_with_name(node, state, sdfg, "Y")
            if len(a.shape) < 2 or len(b.shape) < 2:  # 1-D operands refused (:114-121)
                return False
            return _einsum_can_apply(C.matmul_equation(len(a.shape), len(b.shape)), [a, b], y)
        except Exception:
            return False

    @staticmethod
    def forward(node, state, sdfg):
        a = in_desc_with_name(node, state, sdfg, "A")
        b = in_desc_with_name(node, state, sdfg, "B")
        y = out_desc_with_name(node, state, sdfg, "Y")
        return _einsum_tasklet(node, state, C.matmul_equation(len(a.shape), len(b.shape)), "A", "B", "Y", a, b, y)


@op_implementation(op="Gemm", name=IMPL)
class HipGemm(ONNXForward):
    """PureGemm (pure_implementations.py:380-553): ``Y = alpha * op(A) op(B) + beta * C``, one GEMM launch with alpha
    and C in its epilogue. C is indexed by the trailing letters of the result and its trailing dims must equal Y's
    (:533-539): a vector over the last result index (how nn.Linear exports; ``[1, N]`` is taken as that vector too)
    rides as the column bias, a full ``[M, N]`` matrix as the epilogue's residual operand. ``beta`` other than 0 or 1
    costs one small extra launch: the scaled C (the reference's ``betascale`` map, :540-551) is produced first - a
    vector into the workspace, a matrix into Y, onto which the product is then accumulated."""
    @staticmethod
    def _eq(node):
        a, b = "ik", "kj"
        if node.transA == 1:
            a = a[::-1]
        if node.transB == 1:
            b = b[::-1]
        return "%s,%s->ij" % (a, b)

    @staticmethod
    def _c_kind(c: Array, y: Array) -> Optional[str]:
        """"vector" (C[n] or C[1, n]), "matrix" (C[m, n]) or None (a shape the reference's broadcast rule refuses)."""
        n = y.shape[-1]
        if tuple(c.shape) == tuple(y.shape) and len(y.shape) == 2 and y.shape[0] != 1:
            return "matrix"
        if c.total_size == n and c.shape[-1] == n:
            return "vector"
        return None

    @staticmethod
    def forward_can_be_applied(node, state, sdfg) -> bool:
        try:
            ins, outs = _descs(node, state, sdfg)
            a, b, y = ins["A"], ins["B"], outs["Y"]
            if len(a.shape) != 2 or len(b.shape) != 2:
                return False
            if not _einsum_can_apply(HipGemm._eq(node), [a, b], y):
                return False
            if "C" in ins and node.beta != 0:
                c = ins["C"]
                if not c.is_contiguous() or c.dtype != y.dtype or not y.is_contiguous():
                    return False
                if HipGemm._c_kind(c, y) is None:
                    return False
            return True
        except Exception:
            return False

    @staticmethod
    def forward(node, state, sdfg):
        ins, outs = _descs(node, state, sdfg)
        a, b, y = ins["A"], ins["B"], outs["Y"]
        eq = HipGemm._eq(node)
        if "C" not in ins or node.beta == 0:
            return _einsum_tasklet(node, state, eq, "A", "B", "Y", a, b, y, alpha=node.alpha)
        c = ins["C"]
        kind = HipGemm._c_kind(c, y)
        if node.beta == 1:
            if kind == "vector":
                return _einsum_tasklet(node, state, eq, "A", "B", "Y", a, b, y, alpha=node.alpha, bias="C", bias_desc=c)
            return _einsum_tasklet(node, state, eq, "A", "B", "Y", a, b, y, alpha=node.alpha, residual="C")
        # beta * C first, then the product on top of it
        sfx = _SFX[y.dtype]
        plan = C.plan_contraction(eq, a.shape, a.strides, b.shape, b.strides)
        x_conn, y_conn = ("B", "A") if plan.swapped else ("A", "B")
        if kind == "matrix":
            scale = HipCall("dmlhip_unary_" + sfx, [I32(L.SCALE), Ptr("C"), Ptr("Y"), I64(c.total_size),
                                                    F32(float(node.beta)), Stream()])
            desc = _gemm_struct(plan, node.alpha, 1.0, y.dtype, y.dtype, L.ACT_NONE)
            tail = [Ptr(x_conn), Ptr(y_conn), Ptr("Y"), Null(), Null(), Null()]
            ws, ws_off = 0, 0
        else:
            scale = HipCall("dmlhip_unary_" + sfx, [I32(L.SCALE), Ptr("C"), Workspace(0), I64(c.total_size),
                                                    F32(float(node.beta)), Stream()])
            desc = _gemm_struct(plan, node.alpha, 0.0, y.dtype, c.dtype, L.ACT_NONE)
            ws_off = -(-c.total_size * _ITEMSIZE[c.dtype] // 256) * 256     # the GEMM's own scratch starts past it
            tail = [Ptr(x_conn), Ptr(y_conn), Ptr("Y"), Workspace(0), Null(), Null()]
            ws = ws_off
        if a.dtype == torch.float16:
            import ctypes
            ws += L.load().dmlhip_gemm_f16_workspace_bytes(ctypes.byref(desc))
            gemm = HipCall("dmlhip_gemm_f16_ws", [Struct(desc, "dmlhip_gemm_desc")] + tail +
                           [Workspace(ws_off), WorkspaceBytes(ws_off), Stream()], flops=plan.flops,
                           bytes_moved=_nbytes(a, b, y, c))
        else:
            gemm = HipCall("dmlhip_gemm_f32", [Struct(desc, "dmlhip_gemm_desc")] + tail + [Stream()], flops=plan.flops,
                           bytes_moved=_nbytes(a, b, y, c))
        scale.flops, scale.bytes_moved = 0, 0
        return _tasklet(node, state, [scale, gemm], workspace_bytes=ws, flops=plan.flops,
                        bytes_moved=_nbytes(a, b, y, c), kind="gemm")


# ----------------------------------------------------------------------------- softmax / layernorm
@op_implementation(op="Softmax", name=IMPL)
class HipSoftmax(ONNXForward):
    """Softmax (pure_implementations.py:309-319), opset-12 semantics: everything from ``axis`` on is one
    row. One pass over HBM instead of the four maps and three temporaries of the pure expansion."""
    @staticmethod
    def forward_can_be_applied(node, state, sdfg) -> bool:
        try:
            x = in_desc_with_name(node, state, sdfg, "input")
            y = out_desc_with_name(node, state, sdfg, "output")
            nd = len(x.shape)
            return (_float_ok(x, y) and _dense(x, y) and x.shape == y.shape and nd >= 1
                    and -nd <= node.axis < nd)
        except Exception:
            return False

    @staticmethod
    def forward(node, state, sdfg):
        x = in_desc_with_name(node, state, sdfg, "input")
        axis = node.axis % len(x.shape)
        cols = _prod(x.shape[axis:])
        rows = _prod(x.shape[:axis])
        call = HipCall("dmlhip_softmax_" + _SFX[x.dtype], [Ptr("input"), Ptr("output"), I64(rows), I64(cols), Stream()])
        return _tasklet(node, state, [call], bytes_moved=2 * _nbytes(x), kind="softmax")


@op_implementation(op="LogSoftmax", name=IMPL)
class HipLogSoftmax(ONNXForward):
    """LogSoftmax (pure_implementations.py:649-656), opset-12 semantics like Softmax: everything from ``axis`` on is
    one row. The pure expansion's six statements as six calls on the reduction and elementwise kernels - row maximum,
    ``x - max``, ``exp``, row sum, ``log``, subtraction - with the temporaries in the workspace: the logarithm is
    taken of the row sum, never of a probability, so large negative inputs keep their finite values (a
    ``log(softmax(x))`` would turn everything below the smallest normal into ``-inf``, in fp16 everything below
    about -16)."""
    @staticmethod
    def forward_can_be_applied(node, state, sdfg) -> bool:
        return HipSoftmax.forward_can_be_applied(node, state, sdfg)

    @staticmethod
    def forward(node, state, sdfg):
        x = in_desc_with_name(node, state, sdfg, "input")
        axis = node.axis % len(x.shape)
        rows, cols = _prod(x.shape[:axis]), _prod(x.shape[axis:])
        sfx, code = _SFX[x.dtype], _CODE[x.dtype]
        item = 2 if x.dtype == torch.float16 else 4
        align = lambda n: -(-n // 256) * 256  # noqa: E731
        # workspace: row maxima | x - max | row sums | their logarithms | scratch of the reductions
        o_max, o_sub = 0, align(rows * item)
        o_sum = o_sub + align(rows * cols * item)
        o_log = o_sum + align(rows * item)
        o_scr = o_log + align(rows * item)
        scratch = L.load().dmlhip_reduce_workspace_bytes(rows, cols, 1)
        full, per_row = (rows, cols), (cols, 1)
        reduce = lambda op, src, dst: HipCall(  # noqa: E731
            "dmlhip_reduce_" + sfx, [I32(op), src, dst, I32(code), I64(rows), I64(cols), I64(1), Workspace(o_scr),
                                     WorkspaceBytes(o_scr), Stream()], flops=0, bytes_moved=0)
        sub = lambda a, b, c: HipCall(  # noqa: E731
            "dmlhip_binary_" + sfx, [I32(L.SUB), a, b, c, I32(2), I64Array(full), I64Array(per_row), I64Array((1, 0)),
                                     Stream()], flops=0, bytes_moved=0)
        unary = lambda op, src, dst, n: HipCall(  # noqa: E731
            "dmlhip_unary_" + sfx, [I32(op), src, dst, I64(n), F32(0.0), Stream()], flops=0, bytes_moved=0)
        calls = [reduce(L.RMAX, Ptr("input"), Workspace(o_max)),
                 sub(Ptr("input"), Workspace(o_max), Workspace(o_sub)),
                 unary(L.EXP, Workspace(o_sub), Ptr("output"), rows * cols),       # the output doubles as a temporary
                 reduce(L.RSUM, Ptr("output"), Workspace(o_sum)),
                 unary(L.LOG, Workspace(o_sum), Workspace(o_log), rows),
                 sub(Workspace(o_sub), Workspace(o_log), Ptr("output"))]
        return _tasklet(node, state, calls, workspace_bytes=o_scr + scratch, bytes_moved=8 * _nbytes(x), kind="softmax")


@op_implementation(op="SoftmaxGrad", name=IMPL)
class HipSoftmaxGrad(ONNXForward):
    """The node DefaultSoftmaxBackward builds from ONNXMul / ONNXReduceSum / a subtraction map
    (autodiff/implementations/onnx_ops.py:237-275), as one kernel: dx = y*dy - y*sum(y*dy)."""
    @staticmethod
    def forward_can_be_applied(node, state, sdfg) -> bool:
        try:
            ins, outs = _descs(node, state, sdfg)
            y, dy, dx = ins["Y"], ins["dY"], outs["dX"]
            nd = len(y.shape)
            return (_float_ok(y, dy, dx) and _dense(y, dy, dx) and y.shape == dy.shape == dx.shape
                    and node.axis % nd == nd - 1)
        except Exception:
            return False

    @staticmethod
    def forward(node, state, sdfg):
        y = in_desc_with_name(node, state, sdfg, "Y")
        cols = y.shape[-1]
        rows = _prod(y.shape[:-1])
        call = HipCall("dmlhip_softmax_backward_" + _SFX[y.dtype],
                       [Ptr("Y"), Ptr("dY"), Ptr("dX"), I64(rows), I64(cols), Stream()])
        return _tasklet(node, state, [call], bytes_moved=3 * _nbytes(y), kind="softmax_backward")


def _ln_common(x: Array, gamma: Array, beta: Optional[Array], axis: int) -> bool:
    nd = len(x.shape)
    if nd < 1 or axis % nd != nd - 1:
        return False
    h = x.shape[-1]
    ok = gamma.total_size == h and gamma.is_contiguous() and gamma.dtype == x.dtype
    if beta is not None:
        ok = ok and beta.total_size == h and beta.is_contiguous() and beta.dtype == x.dtype
    return ok


def _stat_ok(d: Optional[Array], rows: int) -> bool:
    return d is None or (d.dtype == torch.float32 and d.is_contiguous() and d.total_size == rows)


@op_implementation(op="LayerNormalization", name=IMPL)
class HipLayerNormalization(ONNXForward):
    """The exporter's nine-node chain ReduceMean, Sub, Pow, ReduceMean, Add, Sqrt, Div, Mul, Add
    (pure_implementations.py:101-103,81-83,39-41,76-78,34-36,91-93), fused by the fusion pass into
    this node and run as one kernel (biased two-pass variance, division by sqrt(var+eps))."""
    @staticmethod
    def forward_can_be_applied(node, state, sdfg) -> bool:
        try:
            ins, outs = _descs(node, state, sdfg)
            x, y = ins["X"], outs["Y"]
            if "B" not in ins or not (_float_ok(x, y) and _dense(x, y) and x.shape == y.shape):
                return False
            rows = _prod(x.shape[:-1])
            return (_ln_common(x, ins["Scale"], ins["B"], node.axis) and _stat_ok(outs.get("Mean"), rows)
                    and _stat_ok(outs.get("InvStdDev"), rows) and node.epsilon >= 0)
        except Exception:
            return False

    @staticmethod
    def forward(node, state, sdfg):
        x = in_desc_with_name(node, state, sdfg, "X")
        rows, cols = _prod(x.shape[:-1]), x.shape[-1]
        call = HipCall("dmlhip_layernorm_" + _SFX[x.dtype],
                       [Ptr("X"), Null(), Ptr("Scale"), Ptr("B"), Ptr("Y"), Null(), _opt(node, state, "Mean", False),
                        _opt(node, state, "InvStdDev", False), I64(rows), I64(cols), F32(node.epsilon), Stream()])
        return _tasklet(node, state, [call], bytes_moved=2 * _nbytes(x), kind="layernorm")


@op_implementation(op="SkipLayerNormalization", name=IMPL)
class HipSkipLayerNormalization(ONNXForward):
    """Residual ONNXAdd (pure_implementations.py:76-78) followed by the LayerNorm chain, in one kernel;
    the sum is rounded to the tensor dtype as the separate Add node would."""
    @staticmethod
    def forward_can_be_applied(node, state, sdfg) -> bool:
        try:
            ins, outs = _descs(node, state, sdfg)
            x, s, y = ins["input"], ins["skip"], outs["output"]
            if "beta" not in ins or not (_float_ok(x, s, y) and _dense(x, s, y) and x.shape == y.shape == s.shape):
                return False
            rows = _prod(x.shape[:-1])
            so = outs.get("input_skip_bias_sum")
            if so is not None and not (so.is_contiguous() and so.shape == x.shape and so.dtype == x.dtype):
                return False
            return (_ln_common(x, ins["gamma"], ins["beta"], -1) and _stat_ok(outs.get("mean"), rows)
                    and _stat_ok(outs.get("inv_std_var"), rows) and node.epsilon >= 0)
        except Exception:
            return False

    @staticmethod
    def forward(node, state, sdfg):
        x = in_desc_with_name(node, state, sdfg, "input")
        rows, cols = _prod(x.shape[:-1]), x.shape[-1]
        has_sum = _has_out(node, state, "input_skip_bias_sum")
        call = HipCall("dmlhip_layernorm_" + _SFX[x.dtype],
                       [Ptr("input"), Ptr("skip"), Ptr("gamma"), Ptr("beta"), Ptr("output"),
                        _opt(node, state, "input_skip_bias_sum", False), _opt(node, state, "mean", False),
                        _opt(node, state, "inv_std_var", False), I64(rows), I64(cols), F32(node.epsilon), Stream()])
        return _tasklet(node, state, [call], bytes_moved=(4 if has_sum else 3) * _nbytes(x), kind="add_layernorm")


@op_implementation(op="LayerNormalizationGrad", name=IMPL)
class HipLayerNormalizationGrad(ONNXForward):
    """Backward of the LayerNorm chain: what the SymPy tasklet reversal plus ReverseReduce
    (autodiff/backward_pass_generator.py:1284-1421, autodiff/implementations/dace_nodes.py:13-105)
    evaluate as a sequence of maps. dX in the tensor dtype, scale/bias gradients in fp32."""
    @staticmethod
    def forward_can_be_applied(node, state, sdfg) -> bool:
        try:
            ins, outs = _descs(node, state, sdfg)
            x, dy, dx = ins["X"], ins["Y_grad"], outs["X_grad"]
            rows, h = _prod(x.shape[:-1]), x.shape[-1]
            if not (_float_ok(x, dy, dx) and _dense(x, dy, dx) and x.shape == dy.shape == dx.shape):
                return False
            for name in ("scale_grad", "bias_grad"):
                d = outs[name]
                if not (d.dtype in (torch.float32, x.dtype) and d.is_contiguous() and d.total_size == h):
                    return False
            return (_ln_common(x, ins["scale"], None, node.axis) and _stat_ok(ins["mean"], rows)
                    and _stat_ok(ins["inv_std_var"], rows))
        except Exception:
            return False

    @staticmethod
    def forward(node, state, sdfg):
        x = in_desc_with_name(node, state, sdfg, "X")
        rows, cols = _prod(x.shape[:-1]), x.shape[-1]
        ws = L.load().dmlhip_layernorm_backward_workspace_bytes(rows, cols)
        gdt = {out_desc_with_name(node, state, sdfg, n).dtype for n in ("scale_grad", "bias_grad")}
        if x.dtype == torch.float16 and gdt == {torch.float16}:
            # both in the tensor dtype (a caller without fp32 master gradients: the reference gives a gradient the dtype
            # of its forward array): the entry point that rounds the fp32 column sums as it stores them
            call = HipCall("dmlhip_layernorm_backward_grads_f16",
                           [Ptr("Y_grad"), Ptr("X"), Ptr("mean"), Ptr("inv_std_var"), Ptr("scale"), Ptr("X_grad"),
                            Ptr("scale_grad"), Ptr("bias_grad"), I32(_CODE[torch.float16]), I64(rows), I64(cols),
                            Workspace(), WorkspaceBytes(), Stream()])
            return _tasklet(node, state, [call], workspace_bytes=ws, bytes_moved=3 * _nbytes(x), kind="layernorm_backward")
        # The kernel sums the scale / shift gradients in fp32 and writes them as fp32. Where the graph wants them in
        # the tensor dtype (a caller without fp32 master gradients: the reference gives a gradient the dtype of its
        # forward array), they land behind the kernel's own workspace and are cast from there.
        grads, casts, end = {}, [], (ws + 255) // 256 * 256
        for name in ("scale_grad", "bias_grad"):
            d = out_desc_with_name(node, state, sdfg, name)
            if d.dtype == torch.float32:
                grads[name] = Ptr(name)
            else:
                grads[name] = Workspace(end)
                casts.append(HipCall("dmlhip_cast", [I32(_CODE[torch.float32]), I32(_CODE[d.dtype]), Workspace(end),
                                                     Ptr(name), I64(cols), Stream()], flops=0, bytes_moved=0))
                end += (cols * 4 + 255) // 256 * 256
        call = HipCall("dmlhip_layernorm_backward_" + _SFX[x.dtype],
                       [Ptr("Y_grad"), Ptr("X"), Ptr("mean"), Ptr("inv_std_var"), Ptr("scale"), Ptr("X_grad"),
                        grads["scale_grad"], grads["bias_grad"], I64(rows), I64(cols), Workspace(), WorkspaceBytes(),
                        Stream()])
        return _tasklet(node, state, [call] + casts, workspace_bytes=end, bytes_moved=3 * _nbytes(x),
                        kind="layernorm_backward")


# ----------------------------------------------------------------------------- elementwise
def _bcast_strides(desc: Array, shape: Sequence[int]) -> Optional[List[int]]:
    nd = len(shape)
    pad = nd - len(desc.shape)
    if pad < 0:
        return None
    out = []
    for i in range(nd):
        if i < pad:
            out.append(0)
            continue
        ext, st = desc.shape[i - pad], desc.strides[i - pad]
        if ext == shape[i]:
            out.append(st if ext != 1 else 0)
        elif ext == 1:
            out.append(0)
        else:
            return None
    return out


def _broadcast_shape(a: Sequence[int], b: Sequence[int]) -> Optional[tuple]:
    nd = max(len(a), len(b))
    a = (1, ) * (nd - len(a)) + tuple(a)
    b = (1, ) * (nd - len(b)) + tuple(b)
    out = []
    for x, y in zip(a, b):
        if x != y and x != 1 and y != 1:
            return None
        out.append(max(x, y) if min(x, y) != 0 else 0)
    return tuple(out)


def _make_binary(op_name: str, code: int, a_conn="A", b_conn="B", c_conn="C"):
    class _Binary(ONNXForward):
        @staticmethod
        def forward_can_be_applied(node, state, sdfg) -> bool:
            try:
                a = in_desc_with_name(node, state, sdfg, a_conn)
                b = in_desc_with_name(node, state, sdfg, b_conn)
                c = out_desc_with_name(node, state, sdfg, c_conn)
                shape = _broadcast_shape(a.shape, b.shape)
                return (_float_ok(a, b, c) and shape is not None and shape == tuple(c.shape) and c.is_contiguous()
                        and len(shape) <= L.MAX_DIMS and a.view_of is None and b.view_of is None)
            except Exception:
                return False

        @staticmethod
        def forward(node, state, sdfg):
            a = in_desc_with_name(node, state, sdfg, a_conn)
            b = in_desc_with_name(node, state, sdfg, b_conn)
            c = out_desc_with_name(node, state, sdfg, c_conn)
            shape = tuple(c.shape)
            call = HipCall("dmlhip_binary_" + _SFX[c.dtype],
                           [I32(code), Ptr(a_conn), Ptr(b_conn), Ptr(c_conn), I32(len(shape)), I64Array(shape),
                            I64Array(tuple(_bcast_strides(a, shape))), I64Array(tuple(_bcast_strides(b, shape))),
                            Stream()])
            return _tasklet(node, state, [call], bytes_moved=_nbytes(a, b, c), kind="elementwise")

    _Binary.__name__ = "Hip" + op_name
    _Binary.__doc__ = ("%s with NumPy broadcasting (pure_implementations.py:39-41,76-93): one vectorised kernel."
                       % op_name)
    return op_implementation(op=op_name, name=IMPL)(_Binary)


HipAdd = _make_binary("Add", L.ADD)
HipSub = _make_binary("Sub", L.SUB)
HipMul = _make_binary("Mul", L.MUL)
HipDiv = _make_binary("Div", L.DIV)
HipPow = _make_binary("Pow", L.POW, "X", "Y", "Z")


def _make_unary(op_name: str, code: int, in_conn: str, out_conn: str, doc: str):
    class _Unary(ONNXForward):
        @staticmethod
        def forward_can_be_applied(node, state, sdfg) -> bool:
            try:
                x = in_desc_with_name(node, state, sdfg, in_conn)
                y = out_desc_with_name(node, state, sdfg, out_conn)
                return _float_ok(x, y) and _dense(x, y) and x.total_size == y.total_size
            except Exception:
                return False

        @staticmethod
        def forward(node, state, sdfg):
            x = in_desc_with_name(node, state, sdfg, in_conn)
            call = HipCall("dmlhip_unary_" + _SFX[x.dtype],
                           [I32(code), Ptr(in_conn), Ptr(out_conn), I64(x.total_size), F32(0.0), Stream()])
            return _tasklet(node, state, [call], bytes_moved=2 * _nbytes(x), kind="elementwise")

    _Unary.__name__ = "Hip" + op_name
    _Unary.__doc__ = doc
    return op_implementation(op=op_name, name=IMPL)(_Unary)


HipSqrt = _make_unary("Sqrt", L.SQRT, "X", "Y", "Sqrt (pure_implementations.py:34-36).")
HipRelu = _make_unary("Relu", L.RELU, "X", "Y", "Relu (pure_implementations.py:556-560).")
HipSigmoid = _make_unary("Sigmoid", L.SIGMOID, "X", "Y", "Sigmoid (pure_implementations.py:741-743).")
HipReciprocal = _make_unary("Reciprocal", L.RECIPROCAL, "X", "Y", "Reciprocal (pure_implementations.py:283-286).")
HipErf = _make_unary("Erf", L.ERF, "input", "output", "Erf (pure_implementations.py:106-108).")
HipExp = _make_unary("Exp", L.EXP, "input", "output", "Exp (pure_implementations.py:29-31).")
HipLog = _make_unary("Log", L.LOG, "input", "output", "Log (pure_implementations.py:24-26).")
HipTanh = _make_unary("Tanh", L.TANH, "input", "output", "Tanh (pure_implementations.py:289-291).")
HipIdentity = _make_unary("Identity", L.IDENTITY, "input", "output", "Identity (pure_implementations.py:255-257).")
HipGelu = _make_unary("Gelu", L.GELU, "X", "Y",
                      "The exporter's Div, Erf, Add, Mul, Mul chain (pure_implementations.py:91-93,106-108,76-78,"
                      "86-88) fused: exact-erf GELU.")
HipSwish = _make_unary("Swish", L.SWISH, "X", "Y", "Mul(x, Sigmoid(x)) (pure_implementations.py:86-88,741-743) fused.")


def _make_unary_grad(op_name: str, code: int, doc: str):
    class _UnaryGrad(ONNXForward):
        @staticmethod
        def forward_can_be_applied(node, state, sdfg) -> bool:
            try:
                ins, outs = _descs(node, state, sdfg)
                x, dy, dx = ins["X"], ins["dY"], outs["dX"]
                return _float_ok(x, dy, dx) and _dense(x, dy, dx) and x.shape == dy.shape == dx.shape
            except Exception:
                return False

        @staticmethod
        def forward(node, state, sdfg):
            x = in_desc_with_name(node, state, sdfg, "X")
            call = HipCall("dmlhip_unary_backward_" + _SFX[x.dtype],
                           [I32(code), Ptr("X"), Ptr("dY"), Ptr("dX"), I64(x.total_size), F32(0.0), Stream()])
            t = _tasklet(node, state, [call], bytes_moved=3 * _nbytes(x), kind="elementwise_backward")
            t.in_place = {"dX": "dY"}   # every thread reads its elements of dY before it writes the same elements of dX
            return t

    _UnaryGrad.__name__ = "Hip" + op_name
    _UnaryGrad.__doc__ = doc
    return op_implementation(op=op_name, name=IMPL)(_UnaryGrad)


_GRAD_DOC = ("dX = dY * f'(X): the tasklet the SymPy reversal of backward_pass_generator.py:1284-1421 derives for "
             "this map, as one kernel.")
HipGeluGrad = _make_unary_grad("GeluGrad", L.GELU, _GRAD_DOC)
HipSwishGrad = _make_unary_grad("SwishGrad", L.SWISH, _GRAD_DOC)
HipSigmoidGrad = _make_unary_grad("SigmoidGrad", L.SIGMOID, _GRAD_DOC)
HipReluGrad = _make_unary_grad("ReluGrad", L.RELU, _GRAD_DOC)
HipTanhGrad = _make_unary_grad("TanhGrad", L.TANH, _GRAD_DOC)
HipErfGrad = _make_unary_grad("ErfGrad", L.ERF, _GRAD_DOC)
HipSqrtGrad = _make_unary_grad("SqrtGrad", L.SQRT, _GRAD_DOC)
HipExpGrad = _make_unary_grad("ExpGrad", L.EXP, _GRAD_DOC)
HipLogGrad = _make_unary_grad("LogGrad", L.LOG, _GRAD_DOC)
HipReciprocalGrad = _make_unary_grad("ReciprocalGrad", L.RECIPROCAL, _GRAD_DOC)


@op_implementation(op="BiasGelu", name=IMPL)
class HipBiasGelu(ONNXForward):
    """Bias ONNXAdd followed by the GELU chain, one kernel."""
    @staticmethod
    def forward_can_be_applied(node, state, sdfg) -> bool:
        try:
            ins, outs = _descs(node, state, sdfg)
            a, b, c = ins["A"], ins["B"], outs["C"]
            return (_float_ok(a, b, c) and _dense(a, b, c) and a.shape == c.shape and len(a.shape) >= 1
                    and b.total_size == a.shape[-1] and b.shape[-1] == a.shape[-1])
        except Exception:
            return False

    @staticmethod
    def forward(node, state, sdfg):
        a = in_desc_with_name(node, state, sdfg, "A")
        rows, cols = _prod(a.shape[:-1]), a.shape[-1]
        call = HipCall("dmlhip_bias_gelu_" + _SFX[a.dtype],
                       [Ptr("A"), Ptr("B"), Ptr("C"), Null(), I64(rows), I64(cols), Stream()])
        return _tasklet(node, state, [call], bytes_moved=2 * _nbytes(a), kind="elementwise")


@op_implementation(op="Sum", name=IMPL)
class HipSum(ONNXForward):
    """PureSum (pure_implementations.py:584-646): all inputs have the output's shape."""
    @staticmethod
    def forward_can_be_applied(node, state, sdfg) -> bool:
        try:
            ins = [sdfg.arrays[e.data.data] for e in node.iter_inputs_in_onnx_order(state)]
            out = out_desc_with_name(node, state, sdfg, "sum")
            return (_float_ok(out, *ins) and _dense(out, *ins) and all(d.shape == out.shape for d in ins)
                    and len(ins) >= 1)
        except Exception:
            return False

    @staticmethod
    def forward(node, state, sdfg):
        conns = [e.dst_conn for e in node.iter_inputs_in_onnx_order(state)]
        out = out_desc_with_name(node, state, sdfg, "sum")
        calls, first, i = [], True, 0
        while i < len(conns):
            chunk = conns[i:i + (8 if first else 7)]
            ptrs = ([] if first else ["sum"]) + chunk
            calls.append(HipCall("dmlhip_sum_" + _SFX[out.dtype],
                                 [PtrArray(tuple(ptrs)), I32(len(ptrs)), Ptr("sum"), I64(out.total_size), Stream()]))
            i += len(chunk)
            first = False
        return _tasklet(node, state, calls, bytes_moved=(len(conns) + 1) * _nbytes(out), kind="elementwise")


@op_implementation(op="Cast", name=IMPL)
class HipCast(ONNXForward):
    """Cast between fp16 and fp32 (pure_implementations.py:329-377)."""
    @staticmethod
    def forward_can_be_applied(node, state, sdfg) -> bool:
        try:
            x = in_desc_with_name(node, state, sdfg, "input")
            y = out_desc_with_name(node, state, sdfg, "output")
            return (x.dtype in FLOAT_DTYPES and y.dtype in FLOAT_DTYPES and _dense(x, y) and x.shape == y.shape)
        except Exception:
            return False

    @staticmethod
    def forward(node, state, sdfg):
        x = in_desc_with_name(node, state, sdfg, "input")
        y = out_desc_with_name(node, state, sdfg, "output")
        call = HipCall("dmlhip_cast", [I32(_CODE[x.dtype]), I32(_CODE[y.dtype]), Ptr("input"), Ptr("output"),
                                       I64(x.total_size), Stream()])
        return _tasklet(node, state, [call], bytes_moved=_nbytes(x, y), kind="elementwise")


# ----------------------------------------------------------------------------- reductions
def _reduce_geometry(shape, axes):
    nd = len(shape)
    axes = sorted(set(range(nd) if axes is None else [a % nd for a in axes]))
    if not axes or axes != list(range(axes[0], axes[-1] + 1)):
        return None
    return _prod(shape[:axes[0]]), _prod(shape[axes[0]:axes[-1] + 1]), _prod(shape[axes[-1] + 1:]), axes


def _reduce_passes(shape, axes):
    """The reduction as a sequence of passes over adjacent axes: [(outer, r, inner)], innermost run of reduced axes
    first (each pass sees the tensor with the runs already reduced collapsed to 1). One pass when the axes are
    adjacent. Sum / Max / Min compose exactly; Mean composes because every pass averages groups of one size."""
    nd = len(shape)
    axes = sorted(set(range(nd) if axes is None else [a % nd for a in axes]))
    if not axes:
        return None
    runs, cur = [], [axes[0]]
    for a in axes[1:]:
        if a == cur[-1] + 1:
            cur.append(a)
        else:
            runs.append(cur)
            cur = [a]
    runs.append(cur)
    shape = list(shape)
    passes = []
    for run in reversed(runs):
        passes.append((_prod(shape[:run[0]]), _prod(shape[run[0]:run[-1] + 1]), _prod(shape[run[-1] + 1:])))
        for a in run:
            shape[a] = 1
    return passes


def _make_reduce(op_name: str, code: int, doc: str):
    class _Reduce(ONNXForward):
        @staticmethod
        def forward_can_be_applied(node, state, sdfg) -> bool:
            try:
                x = in_desc_with_name(node, state, sdfg, "data")
                y = out_desc_with_name(node, state, sdfg, "reduced")
                passes = _reduce_passes(x.shape, node.axes)
                if passes is None or not (x.dtype in FLOAT_DTYPES and y.dtype in FLOAT_DTYPES and _dense(x, y)):
                    return False
                for outer, r, inner in passes:
                    if inner > 1 and outer > 65535:
                        return False
                    if r == 0 and code != L.RSUM:
                        return False
                outer, r, inner = passes[-1]
                return y.total_size == outer * inner
            except Exception:
                return False

        @staticmethod
        def forward(node, state, sdfg):
            x = in_desc_with_name(node, state, sdfg, "data")
            y = out_desc_with_name(node, state, sdfg, "reduced")
            passes = _reduce_passes(x.shape, node.axes)
            lib = L.load()
            if len(passes) == 1:
                outer, r, inner = passes[0]
                ws = lib.dmlhip_reduce_workspace_bytes(outer, r, inner)
                call = HipCall("dmlhip_reduce_" + _SFX[x.dtype],
                               [I32(code), Ptr("data"), Ptr("reduced"), I32(_CODE[y.dtype]), I64(outer), I64(r),
                                I64(inner), Workspace(), WorkspaceBytes(), Stream()])
                return _tasklet(node, state, [call], workspace_bytes=ws, bytes_moved=_nbytes(x, y), kind="reduce")
            # reduced axes that are not adjacent: one pass per run of adjacent axes, innermost run first; results
            # between the passes are fp32 and live in two alternating regions at the head of the workspace, each
            # pass's own scratch behind them
            align = lambda n: -(-n // 256) * 256  # noqa: E731
            region = align(max(o * i for o, _, i in passes[:-1]) * 4)
            scratch = max(lib.dmlhip_reduce_workspace_bytes(o, r, i) for o, r, i in passes)
            calls = []
            for k, (outer, r, inner) in enumerate(passes):
                first, last = k == 0, k == len(passes) - 1
                src = Ptr("data") if first else Workspace(((k - 1) % 2) * region)
                dst = Ptr("reduced") if last else Workspace((k % 2) * region)
                sfx = _SFX[x.dtype] if first else "f32"
                out_code = _CODE[y.dtype] if last else L.F32
                calls.append(HipCall("dmlhip_reduce_" + sfx,
                                     [I32(code), src, dst, I32(out_code), I64(outer), I64(r), I64(inner),
                                      Workspace(2 * region), WorkspaceBytes(2 * region), Stream()],
                                     bytes_moved=_nbytes(x, y) if first else 0, flops=0))
            return _tasklet(node, state, calls, workspace_bytes=2 * region + scratch, bytes_moved=_nbytes(x, y),
                            kind="reduce")

    _Reduce.__name__ = "Hip" + op_name
    _Reduce.__doc__ = doc
    return op_implementation(op=op_name, name=IMPL)(_Reduce)


def _row_split(full, per_row):
    """(rows, cols) when `per_row` is `full` with its trailing axes collapsed to 1, else None."""
    full, per_row = tuple(full), tuple(per_row)
    if len(full) != len(per_row):
        return None
    k = len(full)
    while k > 0 and per_row[k - 1] == 1:
        k -= 1
    if per_row[:k] != full[:k]:
        return None
    return _prod(full[:k]), _prod(full[k:])


@op_implementation(op="RowAffine", name=IMPL)
class HipRowAffine(ONNXForward):
    """Sum (pure_implementations.py:584-646) of Mul(A, per-row S) (:86-88) and a per-row T expanded over the rows and
    scaled (ReverseReduce, autodiff/implementations/dace_nodes.py:13-105) in one pass over A."""
    @staticmethod
    def forward_can_be_applied(node, state, sdfg) -> bool:
        try:
            ins, outs = _descs(node, state, sdfg)
            a, s_, t, y = ins["A"], ins["S"], ins["T"], outs["Y"]
            if not (_float_ok(a, s_, t, y) and a.dtype == s_.dtype == t.dtype == y.dtype and _dense(a, s_, t, y)):
                return False
            if "Scale" in ins and not (ins["Scale"].total_size == 1 and ins["Scale"].dtype == a.dtype):
                return False
            split = _row_split(a.shape, s_.shape)
            return split is not None and split == _row_split(a.shape, t.shape) and tuple(y.shape) == tuple(a.shape)
        except Exception:
            return False

    @staticmethod
    def forward(node, state, sdfg):
        ins, outs = _descs(node, state, sdfg)
        a = ins["A"]
        rows, cols = _row_split(a.shape, ins["S"].shape)
        call = HipCall("dmlhip_row_affine_" + _SFX[a.dtype], [Ptr("A"), Ptr("S"), Ptr("T"), _opt(node, state, "Scale"),
                                                             Ptr("Y"), I64(rows), I64(cols), Stream()])
        return _tasklet(node, state, [call], bytes_moved=2 * _nbytes(a), kind="elementwise")


@op_implementation(op="MulReduceSum", name=IMPL)
class HipMulReduceSum(ONNXForward):
    """Mul (pure_implementations.py:86-88) read only by ReduceSum over the trailing axes (:294-296) as one row-wise dot
    product: the product tensor is never written."""
    @staticmethod
    def forward_can_be_applied(node, state, sdfg) -> bool:
        try:
            a = in_desc_with_name(node, state, sdfg, "A")
            b = in_desc_with_name(node, state, sdfg, "B")
            y = out_desc_with_name(node, state, sdfg, "reduced")
            geo = _reduce_geometry(a.shape, node.axes)
            if geo is None or a.shape != b.shape or not (a.dtype in FLOAT_DTYPES and a.dtype == b.dtype == y.dtype):
                return False
            outer, r, inner, _ = geo
            return inner == 1 and _dense(a, b, y) and y.total_size == outer and outer < 2 ** 31
        except Exception:
            return False

    @staticmethod
    def forward(node, state, sdfg):
        a = in_desc_with_name(node, state, sdfg, "A")
        outer, r, _, _ = _reduce_geometry(a.shape, node.axes)
        call = HipCall("dmlhip_row_dot_" + _SFX[a.dtype], [Ptr("A"), Ptr("B"), Ptr("reduced"), I64(outer), I64(r), Stream()])
        return _tasklet(node, state, [call], flops=2 * a.total_size, bytes_moved=2 * _nbytes(a), kind="reduce")


HipReduceSum = _make_reduce("ReduceSum", L.RSUM, "ReduceSum (pure_implementations.py:294-296).")
HipReduceMax = _make_reduce("ReduceMax", L.RMAX, "ReduceMax (pure_implementations.py:299-301).")
HipReduceMin = _make_reduce("ReduceMin", L.RMIN, "ReduceMin (pure_implementations.py:304-306).")
HipReduceMean = _make_reduce("ReduceMean", L.RMEAN, "ReduceMean (pure_implementations.py:101-103).")


@op_implementation(op="GlobalAveragePool", name=IMPL)
class HipGlobalAveragePool(ONNXForward):
    """GlobalAveragePool "pure" (img_op_implementations.py:415-417): mean over H and W."""
    @staticmethod
    def forward_can_be_applied(node, state, sdfg) -> bool:
        try:
            x = in_desc_with_name(node, state, sdfg, "X")
            y = out_desc_with_name(node, state, sdfg, "Y")
            return (_float_ok(x, y) and _dense(x, y) and len(x.shape) == 4
                    and y.total_size == x.shape[0] * x.shape[1] and x.shape[2] * x.shape[3] > 0)
        except Exception:
            return False

    @staticmethod
    def forward(node, state, sdfg):
        x = in_desc_with_name(node, state, sdfg, "X")
        call = HipCall("dmlhip_reduce_" + _SFX[x.dtype],
                       [I32(L.RMEAN), Ptr("X"), Ptr("Y"), I32(_CODE[x.dtype]), I64(x.shape[0] * x.shape[1]),
                        I64(x.shape[2] * x.shape[3]), I64(1), Null(), USize(0), Stream()])
        return _tasklet(node, state, [call], bytes_moved=_nbytes(x), kind="reduce")


def _pool_geometry(node, x: Array):
    """(kh, kw, sh, sw, oh, ow) of a MaxPool / MaxPoolGrad node over [N, C, H, W]."""
    kh, kw = (int(v) for v in node.kernel_shape)
    sh, sw = (int(v) for v in (node.strides or [1, 1]))
    h, w = x.shape[2], x.shape[3]
    return kh, kw, sh, sw, ((h - kh) // sh + 1 if h >= kh else 0), ((w - kw) // sw + 1 if w >= kw else 0)


@op_implementation(op="MaxPool", name=IMPL)
class HipMaxPool(ONNXForward):
    """PureMaxPool2D (img_op_implementations.py:28-161), with its conditions: two spatial axes, no padding, no dilation,
    no ``Indices`` output, ``ceil_mode`` and ``storage_order`` 0."""
    @staticmethod
    def forward_can_be_applied(node, state, sdfg) -> bool:
        try:
            x = in_desc_with_name(node, state, sdfg, "X")
            y = out_desc_with_name(node, state, sdfg, "Y")
            if _has_out(node, state, "Indices") or len(x.shape) != 4 or not (_float_ok(x, y) and _dense(x, y)):
                return False
            if node.auto_pad != "NOTSET" or node.ceil_mode != 0 or node.storage_order != 0:
                return False
            if len(node.kernel_shape) != 2 or (node.strides is not None and len(node.strides) != 2):
                return False
            if any(p != 0 for p in (node.pads or [])) or any(d != 1 for d in (node.dilations or [])):
                return False
            kh, kw, sh, sw, oh, ow = _pool_geometry(node, x)
            return min(kh, kw, sh, sw) >= 1 and tuple(y.shape) == (x.shape[0], x.shape[1], oh, ow)
        except Exception:
            return False

    @staticmethod
    def forward(node, state, sdfg):
        x = in_desc_with_name(node, state, sdfg, "X")
        y = out_desc_with_name(node, state, sdfg, "Y")
        kh, kw, sh, sw, _, _ = _pool_geometry(node, x)
        call = HipCall("dmlhip_maxpool2d_" + _SFX[x.dtype],
                       [Ptr("X"), Ptr("Y"), I64(x.shape[0] * x.shape[1]), I64(x.shape[2]), I64(x.shape[3]), I64(kh), I64(kw),
                        I64(sh), I64(sw), Stream()])
        return _tasklet(node, state, [call], bytes_moved=_nbytes(x, y), kind="pool")


@op_implementation(op="MaxPoolGrad", name=IMPL)
class HipMaxPoolGrad(ONNXForward):
    """DefaultMaxPoolBackward (autodiff/implementations/onnx_ops.py:284-335) as one kernel: the gradient of each window
    goes to the first position of the window that holds its maximum."""
    @staticmethod
    def forward_can_be_applied(node, state, sdfg) -> bool:
        try:
            ins, outs = _descs(node, state, sdfg)
            x, dy, dx = ins["X"], ins["dY"], outs["dX"]
            if len(x.shape) != 4 or not (_float_ok(x, dy, dx) and _dense(x, dy, dx)) or x.shape != dx.shape:
                return False
            kh, kw, sh, sw, oh, ow = _pool_geometry(node, x)
            return min(kh, kw, sh, sw) >= 1 and tuple(dy.shape) == (x.shape[0], x.shape[1], oh, ow)
        except Exception:
            return False

    @staticmethod
    def forward(node, state, sdfg):
        x = in_desc_with_name(node, state, sdfg, "X")
        dy = in_desc_with_name(node, state, sdfg, "dY")
        kh, kw, sh, sw, _, _ = _pool_geometry(node, x)
        call = HipCall("dmlhip_maxpool2d_backward_" + _SFX[x.dtype],
                       [Ptr("X"), Ptr("dY"), Ptr("dX"), I64(x.shape[0] * x.shape[1]), I64(x.shape[2]), I64(x.shape[3]),
                        I64(kh), I64(kw), I64(sh), I64(sw), Stream()])
        return _tasklet(node, state, [call], bytes_moved=2 * _nbytes(x) + _nbytes(dy), kind="pool")


# ----------------------------------------------------------------------------- data movement
@op_implementation(op="Transpose", name=IMPL)
class HipTranspose(ONNXForward):
    """Transpose (pure_implementations.py:322-326,746-778)."""
    @staticmethod
    def _perm(node, nd):
        return list(reversed(range(nd))) if node.perm is None else [p % nd for p in node.perm]

    @staticmethod
    def forward_can_be_applied(node, state, sdfg) -> bool:
        try:
            x = in_desc_with_name(node, state, sdfg, "data")
            y = out_desc_with_name(node, state, sdfg, "transposed")
            nd = len(x.shape)
            perm = HipTranspose._perm(node, nd)
            return (_float_ok(x, y) and _dense(x, y) and nd <= L.MAX_DIMS and sorted(perm) == list(range(nd))
                    and tuple(x.shape[p] for p in perm) == tuple(y.shape))
        except Exception:
            return False

    @staticmethod
    def forward(node, state, sdfg):
        x = in_desc_with_name(node, state, sdfg, "data")
        perm = HipTranspose._perm(node, len(x.shape))
        call = HipCall("dmlhip_transpose_" + _SFX[x.dtype],
                       [Ptr("data"), Ptr("transposed"), I32(len(perm)), I64Array(tuple(x.shape)), I64Array(tuple(perm)),
                        Stream()])
        return _tasklet(node, state, [call], bytes_moved=2 * _nbytes(x), kind="transpose")


@op_implementation(op="Pad", name=IMPL)
class HipPad(ONNXForward):
    """Pad with a constant (the node's attribute form: the importer has turned the ``pads`` / ``constant_value``
    inputs into attributes). Negative amounts crop, which is how the node's own reverse is expressed. The reference
    has no expansion for Pad; in front of a Conv the fusion pass removes it (fuse_pad_into_conv)."""
    @staticmethod
    def forward_can_be_applied(node, state, sdfg) -> bool:
        try:
            x = in_desc_with_name(node, state, sdfg, "data")
            y = out_desc_with_name(node, state, sdfg, "output")
            nd = len(x.shape)
            pads = [int(p) for p in node.pads]
            return (node.mode == "constant" and _float_ok(x, y) and _dense(x, y) and nd <= L.MAX_DIMS
                    and len(pads) == 2 * nd
                    and tuple(y.shape) == tuple(d + pads[i] + pads[nd + i] for i, d in enumerate(x.shape)))
        except Exception:
            return False

    @staticmethod
    def forward(node, state, sdfg):
        x = in_desc_with_name(node, state, sdfg, "data")
        y = out_desc_with_name(node, state, sdfg, "output")
        nd = len(x.shape)
        pads = [int(p) for p in node.pads]
        call = HipCall("dmlhip_pad_constant_" + _SFX[x.dtype],
                       [Ptr("data"), Ptr("output"), I32(nd), I64Array(tuple(x.shape)), I64Array(tuple(pads[:nd])),
                        I64Array(tuple(pads[nd:])), F32(float(node.value)), Stream()])
        return _tasklet(node, state, [call], bytes_moved=_nbytes(x) + _nbytes(y), kind="elementwise")


@op_implementation(op="Reshape", name=IMPL)
class HipReshape(ONNXForward):
    """Reshape (pure_implementations.py:571-573): a dense copy into the output descriptor."""
    @staticmethod
    def forward_can_be_applied(node, state, sdfg) -> bool:
        try:
            x = in_desc_with_name(node, state, sdfg, "data")
            y = out_desc_with_name(node, state, sdfg, "reshaped")
            return _float_ok(x, y) and _dense(x, y) and x.total_size == y.total_size
        except Exception:
            return False

    @staticmethod
    def forward(node, state, sdfg):
        x = in_desc_with_name(node, state, sdfg, "data")
        call = HipCall("dmlhip_unary_" + _SFX[x.dtype],
                       [I32(L.IDENTITY), Ptr("data"), Ptr("reshaped"), I64(x.total_size), F32(0.0), Stream()])
        return _tasklet(node, state, [call], bytes_moved=2 * _nbytes(x), kind="elementwise")


# ----------------------------------------------------------------------------- batch normalisation
def _bn_ok(x, *vectors) -> bool:
    if len(x.shape) < 2 or not (_float_ok(x) and _dense(x)):
        return False
    return all(v.dtype == x.dtype and v.is_contiguous() and v.total_size == x.shape[1] for v in vectors)


def _bn_dims(x):
    n, c = x.shape[0], x.shape[1]
    return n, c, x.total_size // max(n * c, 1)


@op_implementation(op="BatchNormalization", name=IMPL)
class HipBatchNormalization(ONNXForward):
    """Inference (only Y connected) and training (all five outputs connected) forms of PureBatchNormalization
    (img_op_implementations.py:333-412; cuDNN variant cudnn_implementations.py:444-649): biased batch variance,
    running statistics updated as ``in * momentum + saved * (1 - momentum)``. As in the reference (:392-410) the
    updated running statistics are also written back to the arrays they came from, when those are caller-owned
    buffers. A private ``_activation`` attribute ("relu" / "swish") set by the fusion pass applies a following
    activation in the same kernel."""
    @staticmethod
    def forward_can_be_applied(node, state, sdfg) -> bool:
        try:
            ins, outs = _descs(node, state, sdfg)
            x, y = ins["X"], outs["Y"]
            if getattr(node, "_activation", "none") not in ("none", "relu", "swish"):
                return False
            stats = [outs.get(k) for k in ("out_mean", "out_var", "saved_mean", "saved_var")]
            if any(s is None for s in stats) and any(s is not None for s in stats):
                return False
            return (_dense(y) and y.shape == x.shape and y.dtype == x.dtype and node.epsilon >= 0
                    and _bn_ok(x, ins["scale"], ins["B"], ins["in_mean"], ins["in_var"], *[s for s in stats if s]))
        except Exception:
            return False

    @staticmethod
    def forward(node, state, sdfg):
        x = in_desc_with_name(node, state, sdfg, "X")
        n, c, hw = _bn_dims(x)
        sfx = _SFX[x.dtype]
        training = "saved_mean" in {e.src_conn for e in state.out_edges(node)}
        act = getattr(node, "_activation", "none")
        fused = [] if act == "none" else [I32(_ACT[act])]
        variant = "" if act == "none" else "act_"
        if not training:
            call = HipCall("dmlhip_batchnorm_inference_" + variant + sfx,
                           [Ptr("X"), Ptr("scale"), Ptr("B"), Ptr("in_mean"), Ptr("in_var"), Ptr("Y"), I64(n), I64(c),
                            I64(hw), F32(node.epsilon)] + fused + [Stream()])
            return _tasklet(node, state, [call], bytes_moved=2 * _nbytes(x), kind="batchnorm")
        ws = L.load().dmlhip_batchnorm_workspace_bytes(n, c, hw)
        # running statistics: where the updated value has no reader of its own and the array it came from is a
        # caller-owned buffer, the kernel writes it there directly (its out_* may alias its in_*); otherwise it goes to
        # the node's output and, for caller-owned inputs, is copied back as the reference does (:392-410)
        out_ptr, copies = {}, []
        for src, dst in (("out_mean", "in_mean"), ("out_var", "in_var")):
            in_arr = next(iter(state.in_edges_by_connector(node, dst))).data.data
            out_arr = next(iter(state.out_edges_by_connector(node, src))).data.data
            caller_owned = not sdfg.arrays[in_arr].transient and in_arr not in sdfg.constants
            unread = (sdfg.arrays[out_arr].transient
                      and not any(isinstance(e.src, AccessNode) and e.src.data == out_arr
                                  for st in sdfg.states() for e in st.edges())
                      and not any(d.view_of == out_arr for d in sdfg.arrays.values()))
            out_ptr[src] = Ptr(dst) if (caller_owned and unread) else Ptr(src)
            if caller_owned and not unread:
                copies.append(HipCall("dmlhip_unary_" + sfx, [I32(L.IDENTITY), Ptr(src), Ptr(dst), I64(c), F32(0.0),
                                                              Stream()]))
        calls = [HipCall("dmlhip_batchnorm_training_" + variant + sfx,
                         [Ptr("X"), Ptr("scale"), Ptr("B"), Ptr("in_mean"), Ptr("in_var"), Ptr("Y"), out_ptr["out_mean"],
                          out_ptr["out_var"], Ptr("saved_mean"), Ptr("saved_var"), I64(n), I64(c), I64(hw),
                          F32(node.epsilon), F32(node.momentum)] + fused + [Workspace(), WorkspaceBytes(), Stream()])]
        calls += copies
        return _tasklet(node, state, calls, workspace_bytes=ws, bytes_moved=3 * _nbytes(x), kind="batchnorm")


@op_implementation(op="BatchNormalizationGrad", name=IMPL)
class HipBatchNormalizationGrad(ONNXForward):
    """Backward of training-mode BatchNormalization (CuDNNBatchNormBackward,
    autodiff/implementations/onnx_ops.py:1268-1510): dX in the tensor type, dscale / dB in fp32."""
    @staticmethod
    def forward_can_be_applied(node, state, sdfg) -> bool:
        try:
            ins, outs = _descs(node, state, sdfg)
            x, dy = ins["X"], ins["dY"]
            if not (_bn_ok(x, ins["scale"], ins["saved_mean"], ins["saved_var"]) and _dense(dy)
                    and dy.shape == x.shape and dy.dtype == x.dtype and outs):
                return False
            if node.activation not in ("none", "relu", "swish"):
                return False
            if node.activation != "none" and not ("B" in ins and _bn_ok(x, ins["B"])):
                return False
            dx = outs.get("dX")
            if dx is not None and not (_dense(dx) and dx.shape == x.shape and dx.dtype == x.dtype):
                return False
            return all(d is None or (d.dtype == torch.float32 and d.is_contiguous() and d.total_size == x.shape[1])
                       for d in (outs.get("dscale"), outs.get("dB")))
        except Exception:
            return False

    @staticmethod
    def forward(node, state, sdfg):
        x = in_desc_with_name(node, state, sdfg, "X")
        n, c, hw = _bn_dims(x)
        ws = L.load().dmlhip_batchnorm_workspace_bytes(n, c, hw)
        fused = node.activation != "none"
        call = HipCall("dmlhip_batchnorm_backward_" + ("act_" if fused else "") + _SFX[x.dtype],
                       [Ptr("dY"), Ptr("X"), Ptr("scale")] + ([Ptr("B")] if fused else []) +
                       [Ptr("saved_mean"), Ptr("saved_var"), _opt(node, state, "dX", False),
                        _opt(node, state, "dscale", False), _opt(node, state, "dB", False), I64(n), I64(c), I64(hw),
                        F32(node.epsilon)] + ([I32(_ACT[node.activation])] if fused else []) +
                       [Workspace(), WorkspaceBytes(), Stream()])
        return _tasklet(node, state, [call], workspace_bytes=ws, bytes_moved=5 * _nbytes(x), kind="batchnorm_backward")


# ----------------------------------------------------------------------------- convolution
def _conv_struct(node, x: Array, w: Array, act=L.ACT_NONE) -> Optional[L.Conv2dDesc]:
    """Attribute handling of CudnnConvolution (cudnn_implementations.py:148-275): 1-D and 2-D, symmetric pads,
    auto_pad NOTSET, any stride / dilation / group. A 1-D convolution over [N, C, L] is the 2-D one over [N, C, 1, L]
    with a 1 x k filter (the reference hands cuDNN [N, C, L, 1] and a k x 1 filter, :243-250; the dense tensors are
    the same bytes either way, and a row of L contiguous elements is what these kernels stream)."""
    nsp = len(x.shape) - 2
    if nsp not in (1, 2) or len(w.shape) != len(x.shape) or node.auto_pad != "NOTSET":
        return None
    strides = list(node.strides) if node.strides is not None else [1] * nsp
    dil = list(node.dilations) if node.dilations is not None else [1] * nsp
    pads = list(node.pads) if node.pads is not None else [0] * (2 * nsp)
    if len(strides) != nsp or len(dil) != nsp or len(pads) != 2 * nsp:
        return None
    if any(pads[i] != pads[nsp + i] for i in range(nsp)):
        return None
    if node.kernel_shape is not None and list(node.kernel_shape) != list(w.shape[2:]):
        return None
    group = int(node.group)
    if group < 1 or x.shape[1] != w.shape[1] * group or w.shape[0] % group:
        return None
    if nsp == 1:
        strides, dil, pads = [1] + strides, [1] + dil, [0, pads[0], 0, pads[1]]
    d = L.Conv2dDesc()
    d.n, d.c = x.shape[0], x.shape[1]
    d.h, d.w = (1, x.shape[2]) if nsp == 1 else x.shape[2:]
    d.m = w.shape[0]
    d.kh, d.kw = (1, w.shape[2]) if nsp == 1 else w.shape[2:]
    d.stride_h, d.stride_w = strides
    d.pad_h, d.pad_w = pads[0], pads[1]
    d.dil_h, d.dil_w = dil
    d.group = group
    d.act = act
    return d


def _tensor_layout(desc: Array) -> Optional[str]:
    """"NCHW", "NHWC" or None for a 3-D / 4-D tensor whose shape is in ONNX order [N, C, spatial..]: the test of
    ``_get_tensor_layout`` (cudnn_implementations.py:20-66) - the strides are those of the dense tensor, or those of
    a dense channels-last tensor viewed in ONNX order. Where the two coincide (one channel, or one pixel) it is NCHW."""
    shape, strides = tuple(desc.shape), tuple(desc.strides)
    if len(shape) not in (3, 4):
        return None
    if desc.is_contiguous():
        return "NCHW"
    last = shape[:1] + shape[2:] + shape[1:2]                # the channels-last shape
    dense = [_prod(last[i + 1:]) for i in range(len(last))]  # and its dense strides
    as_onnx = tuple(dense[:1] + dense[-1:] + dense[1:-1])
    relevant = [i for i in range(len(shape)) if shape[i] > 1]
    return "NHWC" if all(strides[i] == as_onnx[i] for i in relevant) else None


def _conv_out_shape(d: L.Conv2dDesc, x: Array):
    """Shape of Y for the descriptor `_conv_struct` made from X (three dimensions for a 1-D convolution)."""
    oh, ow = _conv_out_hw(d)
    return (d.n, d.m, ow) if len(x.shape) == 3 else (d.n, d.m, oh, ow)


def _conv_out_hw(d: L.Conv2dDesc):
    eh = (d.kh - 1) * d.dil_h + 1
    ew = (d.kw - 1) * d.dil_w + 1
    oh = (d.h + 2 * d.pad_h - eh) // d.stride_h + 1 if d.h + 2 * d.pad_h >= eh else 0
    ow = (d.w + 2 * d.pad_w - ew) // d.stride_w + 1 if d.w + 2 * d.pad_w >= ew else 0
    return oh, ow


@op_implementation(op="Conv", name=IMPL)
class HipConv(ONNXForward):
    """ONNX Conv. PureConv2D (img_op_implementations.py:164-330) covers stride 1 / no pad / group 1 only
    and the reference otherwise needs cuDNN or ONNX Runtime; this covers strides, symmetric pads,
    dilations and groups: 1x1 as an MFMA GEMM, depthwise from LDS-staged rows, the rest directly.
    A private ``_activation`` attribute set by the fusion pass folds a following Swish / Sigmoid in."""
    @staticmethod
    def forward_can_be_applied(node, state, sdfg) -> bool:
        try:
            ins, outs = _descs(node, state, sdfg)
            x, w, y = ins["X"], ins["W"], outs["Y"]
            if not (_float_ok(x, w, y) and _dense(w)) or _tensor_layout(x) is None or _tensor_layout(y) is None:
                return False
            if "B" in ins and not (ins["B"].dtype == x.dtype and ins["B"].is_contiguous()
                                   and ins["B"].total_size == w.shape[0]):
                return False
            d = _conv_struct(node, x, w)
            if d is None:
                return False
            return tuple(y.shape) == _conv_out_shape(d, x)
        except Exception:
            return False

    @staticmethod
    def forward(node, state, sdfg):
        """One call for dense NCHW tensors. A channels-last X or Y (ONNX-order shape, NHWC strides: what
        CudnnConvolution passes to cuDNN as CUDNN_TENSOR_NHWC, cudnn_implementations.py:69-110) is brought into the
        kernels' layout by a transpose into the workspace before, respectively out of it after, the convolution."""
        ins, outs = _descs(node, state, sdfg)
        x, w, y = ins["X"], ins["W"], outs["Y"]
        d = _conv_struct(node, x, w, _ACT[getattr(node, "_activation", "none")])
        sfx = _SFX[x.dtype]
        calls, ws = [], 0
        x_arg, y_arg = Ptr("X"), Ptr("Y")
        if _tensor_layout(x) == "NHWC":
            last = tuple(x.shape[:1]) + tuple(x.shape[2:]) + tuple(x.shape[1:2])
            back = (0, len(last) - 1) + tuple(range(1, len(last) - 1))
            calls.append(HipCall("dmlhip_transpose_" + sfx, [Ptr("X"), Workspace(0), I32(len(last)), I64Array(last),
                                                             I64Array(back), Stream()], flops=0, bytes_moved=2 * _nbytes(x)))
            x_arg = Workspace(0)
            ws = (_nbytes(x) + 255) // 256 * 256
        y_nhwc = _tensor_layout(y) == "NHWC"
        if y_nhwc:
            y_arg = Workspace(ws)
        flops = 2 * y.total_size * int(math.prod(w.shape[1:]))
        calls.append(HipCall("dmlhip_conv2d_" + sfx, [Struct(d, "dmlhip_conv2d_desc"), x_arg, Ptr("W"), _opt(node, state, "B"),
                                                      y_arg, Stream()], flops=flops, bytes_moved=_nbytes(x, w, y)))
        if y_nhwc:
            nd = len(y.shape)
            calls.append(HipCall("dmlhip_transpose_" + sfx, [Workspace(ws), Ptr("Y"), I32(nd), I64Array(tuple(y.shape)),
                                                             I64Array((0, ) + tuple(range(2, nd)) + (1, )), Stream()],
                                 flops=0, bytes_moved=2 * _nbytes(y)))
            ws += (_nbytes(y) + 255) // 256 * 256
        return _tasklet(node, state, calls, workspace_bytes=ws, flops=flops, bytes_moved=_nbytes(x, w, y), kind="conv")


@op_implementation(op="GatedConv", name=IMPL)
class HipGatedConv(ONNXForward):
    """Mul(X, Gate[n, c, 1, 1]) followed by a pointwise Conv (pure_implementations.py:86-88 +
    img_op_implementations.py:164-330) in one kernel: the gate scales X on its way into LDS. fp32."""
    @staticmethod
    def forward_can_be_applied(node, state, sdfg) -> bool:
        try:
            ins, outs = _descs(node, state, sdfg)
            x, gt, w, y = ins["X"], ins["Gate"], ins["W"], outs["Y"]
            if x.dtype != torch.float32 or not (_float_ok(x, gt, w, y) and _dense(x, gt, w, y)):
                return False
            if tuple(gt.shape) != (x.shape[0], x.shape[1], 1, 1) or tuple(w.shape[2:]) != (1, 1):
                return False
            if "B" in ins and not (ins["B"].dtype == x.dtype and ins["B"].is_contiguous()
                                   and ins["B"].total_size == w.shape[0]):
                return False
            d = _conv_struct(node, x, w)
            if d is None or (d.stride_h, d.stride_w, d.pad_h, d.pad_w, d.group) != (1, 1, 0, 0, 1):
                return False
            hw = x.shape[2] * x.shape[3]
            return (x.shape[1] % 32 == 0 and hw % 4 == 0 and hw >= 128 and x.shape[0] <= 65535
                    and tuple(y.shape) == (x.shape[0], w.shape[0], x.shape[2], x.shape[3]))
        except Exception:
            return False

    @staticmethod
    def forward(node, state, sdfg):
        ins, outs = _descs(node, state, sdfg)
        x, w, y = ins["X"], ins["W"], outs["Y"]
        d = _conv_struct(node, x, w, _ACT[getattr(node, "_activation", "none")])
        call = HipCall("dmlhip_conv2d_gated_f32", [Struct(d, "dmlhip_conv2d_desc"), Ptr("X"), Ptr("Gate"), Ptr("W"),
                                                   _opt(node, state, "B"), Ptr("Y"), Stream()])
        return _tasklet(node, state, [call], flops=2 * y.total_size * w.shape[1] + x.total_size,
                        bytes_moved=_nbytes(x, ins["Gate"], w, y), kind="conv")


@op_implementation(op="ExpandDepthwiseConv", name=IMPL)
class HipExpandDepthwiseConv(ONNXForward):
    """Pointwise Conv + activation + 3x3 depthwise Conv + activation (img_op_implementations.py:164-330 twice, with
    the elementwise ops of pure_implementations.py:556-560 between) in one kernel; the expanded tensor stays in LDS.
    fp32."""
    @staticmethod
    def _descs(node, x, w_pw, w_dw, y):
        stride = int((node.strides or [1, 1])[0])
        mid = (x.shape[0], w_pw.shape[0], x.shape[2], x.shape[3])
        pw, dw = L.Conv2dDesc(), L.Conv2dDesc()
        pw.n, pw.c, pw.h, pw.w = x.shape
        pw.m, pw.kh, pw.kw = w_pw.shape[0], 1, 1
        pw.stride_h = pw.stride_w = pw.dil_h = pw.dil_w = pw.group = 1
        pw.pad_h = pw.pad_w = 0
        pw.act = _ACT[node.act_pw]
        dw.n, dw.c, dw.h, dw.w = mid
        dw.m, dw.kh, dw.kw = mid[1], 3, 3
        dw.stride_h = dw.stride_w = stride
        dw.pad_h = dw.pad_w = dw.dil_h = dw.dil_w = 1
        dw.group = mid[1]
        dw.act = _ACT[node.act_dw]
        oh, ow = (x.shape[2] - 1) // stride + 1, (x.shape[3] - 1) // stride + 1
        return pw, dw, (x.shape[0], w_pw.shape[0], oh, ow)

    @staticmethod
    def forward_can_be_applied(node, state, sdfg) -> bool:
        try:
            ins, outs = _descs(node, state, sdfg)
            x, w1, w2, y = ins["X"], ins["W_pw"], ins["W_dw"], outs["Y"]
            if x.dtype != torch.float32 or not (_float_ok(x, w1, w2, y) and _dense(x, w1, w2, y)):
                return False
            if len(x.shape) != 4 or tuple(w1.shape) != (w1.shape[0], x.shape[1], 1, 1):
                return False
            if tuple(w2.shape) != (w1.shape[0], 1, 3, 3) or list(node.strides or [1, 1]) not in ([1, 1], [2, 2]):
                return False
            for b in ("B_pw", "B_dw"):
                if b in ins and not (ins[b].dtype == x.dtype and ins[b].is_contiguous()
                                     and ins[b].total_size == w1.shape[0]):
                    return False
            from daceml_amd.transformation.fusion import EXPAND_DEPTHWISE_ACTIVATIONS
            if (node.act_pw, node.act_dw) not in EXPAND_DEPTHWISE_ACTIVATIONS:
                return False
            _, _, yshape = HipExpandDepthwiseConv._descs(node, x, w1, w2, y)
            return (x.shape[1] % 16 == 0 and w1.shape[0] % 32 == 0 and tuple(y.shape) == yshape
                    and 32 * 3 * (x.shape[3] + 2) * 4 <= 140 * 1024)
        except Exception:
            return False

    @staticmethod
    def forward(node, state, sdfg):
        ins, outs = _descs(node, state, sdfg)
        x, w1, w2, y = ins["X"], ins["W_pw"], ins["W_dw"], outs["Y"]
        pw, dw, _ = HipExpandDepthwiseConv._descs(node, x, w1, w2, y)
        call = HipCall("dmlhip_conv2d_expand_depthwise_f32",
                       [Struct(pw, "dmlhip_conv2d_desc"), Struct(dw, "dmlhip_conv2d_desc"), Ptr("X"), Ptr("W_pw"),
                        _opt(node, state, "B_pw"), Ptr("W_dw"), _opt(node, state, "B_dw"), Ptr("Y"), Stream()])
        mid = x.shape[0] * w1.shape[0] * x.shape[2] * x.shape[3]
        return _tasklet(node, state, [call], flops=2 * mid * x.shape[1] + 18 * y.total_size,
                        bytes_moved=_nbytes(x, w1, w2, y), kind="conv")


@op_implementation(op="ConvGrad", name=IMPL)
class HipConvGrad(ONNXForward):
    """cudnnConvolutionBackwardData / BackwardFilter / BackwardBias
    (autodiff/implementations/onnx_ops.py:663-703) and the ATen depthwise backward (:1201-1231); fp32."""
    @staticmethod
    def forward_can_be_applied(node, state, sdfg) -> bool:
        try:
            ins, outs = _descs(node, state, sdfg)
            x, w, dy = ins["X"], ins["W"], ins["dY"]
            if x.dtype != torch.float32 or not (_float_ok(x, w, dy) and _dense(x, w, dy)):
                return False
            d = _conv_struct(node, x, w)
            if d is None:
                return False
            if tuple(dy.shape) != _conv_out_shape(d, x):
                return False
            for name, ref in (("dX", x), ("dW", w)):
                if name in outs and not (outs[name].shape == ref.shape and outs[name].is_contiguous()
                                         and outs[name].dtype == torch.float32):
                    return False
            if "dB" in outs and not (outs["dB"].total_size == w.shape[0] and outs["dB"].dtype == torch.float32):
                return False
            return x.shape[0] <= 65535
        except Exception:
            return False

    @staticmethod
    def forward(node, state, sdfg):
        ins, outs = _descs(node, state, sdfg)
        x, w, dy = ins["X"], ins["W"], ins["dY"]
        d = _conv_struct(node, x, w)
        lib = L.load()
        calls, ws = [], 0
        work = 2 * dy.total_size * int(math.prod(w.shape[1:]))     # of each of the two gradients
        if "dX" in outs:
            calls.append(HipCall("dmlhip_conv2d_backward_data_f32",
                                 [Struct(d, "dmlhip_conv2d_desc"), Ptr("dY"), Ptr("W"), Ptr("dX"), Stream()],
                                 flops=work, bytes_moved=_nbytes(dy, w, x)))
        if "dW" in outs:
            import ctypes
            ws = max(ws, lib.dmlhip_conv2d_backward_weight_workspace_bytes(ctypes.byref(d)))
            calls.append(HipCall("dmlhip_conv2d_backward_weight_f32",
                                 [Struct(d, "dmlhip_conv2d_desc"), Ptr("X"), Ptr("dY"), Ptr("dW"), Workspace(),
                                  WorkspaceBytes(), Stream()], flops=work, bytes_moved=_nbytes(x, dy, w)))
        if "dB" in outs:
            # dB[m] = sum_{b, y, x} dY[b, m, y, x]: reduce the spatial dims into the head of the
            # workspace, then the batch dim from there
            n, m = dy.shape[0], dy.shape[1]
            hw = int(math.prod(dy.shape[2:]))
            part = (n * m * 4 + 255) // 256 * 256
            ws = max(ws, part + lib.dmlhip_reduce_workspace_bytes(1, n, m))
            calls.append(HipCall("dmlhip_reduce_f32", [I32(L.RSUM), Ptr("dY"), Workspace(), I32(L.F32), I64(n * m),
                                                       I64(hw), I64(1), Null(), USize(0), Stream()]))
            calls.append(HipCall("dmlhip_reduce_f32", [I32(L.RSUM), Workspace(), Ptr("dB"), I32(L.F32), I64(1), I64(n),
                                                       I64(m), Workspace(part), WorkspaceBytes(part), Stream()]))
        return _tasklet(node, state, calls, workspace_bytes=ws, bytes_moved=_nbytes(x, w, dy), kind="conv_backward")


# ----------------------------------------------------------------------------- fused attention
def _attn_struct(perm_descs, q: Array, k: Array, scale: float, q_perm, k_perm) -> L.AttentionDesc:
    """perm_descs: four (descriptor, perm) pairs in the q / k / v / o slots of dmlhip_attention_desc."""
    d = L.AttentionDesc()
    for i in (0, 1):
        d.batch[i] = 1 if q_perm[i] < 0 else int(q.shape[q_perm[i]])
    d.seq_q, d.seq_k, d.head_dim = int(q.shape[q_perm[2]]), int(k.shape[k_perm[2]]), int(q.shape[q_perm[3]])
    for name, (desc, perm) in zip(("q_stride", "k_stride", "v_stride", "o_stride"), perm_descs):
        for i in range(3):
            getattr(d, name)[i] = 0 if perm[i] < 0 else int(desc.strides[perm[i]])
    d.scale = float(scale)
    return d


def _attn_ok(node, descs_perms) -> bool:
    """Shapes of the four tensors agree with each other and with what the kernel covers."""
    (q, qp), (k, kp), (v, vp), (o, op_) = descs_perms
    for d, pm in descs_perms:
        if d.dtype != torch.float16 or len(pm) != 4 or d.shape[pm[3]] != 64 or d.strides[pm[3]] != 1:
            return False
        if any(pm[i] >= 0 and d.strides[pm[i]] % 8 for i in range(3)):
            return False
        if sorted(i for i in pm if i >= 0) != list(range(len(d.shape))):
            return False

    def ext(d, pm, i):
        return 1 if pm[i] < 0 else d.shape[pm[i]]

    for i in (0, 1):
        if len({ext(q, qp, i), ext(k, kp, i), ext(v, vp, i), ext(o, op_, i)}) != 1:
            return False
    return ext(k, kp, 2) == ext(v, vp, 2) and ext(q, qp, 2) == ext(o, op_, 2) and ext(k, kp, 2) > 0


def attention_mask_strides(mask: Array, q: Array, k: Array, q_perm, k_perm) -> Optional[Tuple[int, int]]:
    """Element strides of an additive mask over (batch0, batch1), or None when the kernels cannot take it. The mask
    broadcasts against the scores [batch.., queries, keys] by Add's right-aligned rule (pure_implementations.py:34-36
    is NumPy's); the kernels want fp16, one contiguous row of keys per batch entry and no dependence on the query."""
    ext = [1 if q_perm[i] < 0 else q.shape[q_perm[i]] for i in (0, 1)] + [q.shape[q_perm[2]], k.shape[k_perm[2]]]
    nd = 2 + sum(1 for i in (0, 1) if q_perm[i] >= 0)
    if mask.dtype != torch.float16 or len(mask.shape) > nd:
        return None
    shape = [1] * (4 - len(mask.shape)) + list(mask.shape)
    strides = [0] * (4 - len(mask.shape)) + list(mask.strides)
    if shape[3] != ext[3] or (shape[3] > 1 and strides[3] != 1) or (shape[2] != 1 and ext[2] != 1):
        return None
    out = []
    for i in (0, 1):
        if shape[i] == 1:
            out.append(0)
        elif shape[i] == ext[i] and strides[i] % 4 == 0:
            out.append(int(strides[i]))
        else:
            return None
    return out[0], out[1]


@op_implementation(op="FusedAttention", name=IMPL)
class HipFusedAttention(ONNXForward):
    """softmax(scale * Q K^T) V in one kernel: the composition of PureEinsum (pure_implementations.py:219-252),
    the scalar Mul (:86-88), Softmax over the last axis (:309-319) and a second PureEinsum, without the score
    matrix in memory. Optional output LogSumExp (fp32, [batch0, batch1, seq_q]) is what the backward node needs
    instead of the probabilities."""
    @staticmethod
    def _pairs(node, ins, outs):
        return [(ins["Q"], node.q_perm), (ins["K"], node.k_perm), (ins["V"], node.v_perm), (outs["Output"], node.o_perm)]

    @staticmethod
    def forward_can_be_applied(node, state, sdfg) -> bool:
        try:
            ins, outs = _descs(node, state, sdfg)
            if not _attn_ok(node, HipFusedAttention._pairs(node, ins, outs)):
                return False
            if "Mask" in ins and attention_mask_strides(ins["Mask"], ins["Q"], ins["K"], node.q_perm, node.k_perm) is None:
                return False
            lse = outs.get("LogSumExp")
            return lse is None or (lse.dtype == torch.float32 and lse.is_contiguous())
        except Exception:
            return False

    @staticmethod
    def forward(node, state, sdfg):
        ins, outs = _descs(node, state, sdfg)
        pairs = HipFusedAttention._pairs(node, ins, outs)
        d = _attn_struct(pairs, ins["Q"], ins["K"], node.scale, node.q_perm, node.k_perm)
        if "Mask" in ins:
            ms = attention_mask_strides(ins["Mask"], ins["Q"], ins["K"], node.q_perm, node.k_perm)
            call = HipCall("dmlhip_attention_masked_f16",
                           [Struct(d, "dmlhip_attention_desc"), Ptr("Q"), Ptr("K"), Ptr("V"), Ptr("Mask"), I64Array(ms),
                            Ptr("Output"), _opt(node, state, "LogSumExp", False), Stream()])
        else:
            call = HipCall("dmlhip_attention_f16", [Struct(d, "dmlhip_attention_desc"), Ptr("Q"), Ptr("K"), Ptr("V"),
                                                    Ptr("Output"), _opt(node, state, "LogSumExp", False), Stream()])
        bh = d.batch[0] * d.batch[1]
        return _tasklet(node, state, [call], flops=4 * bh * d.seq_q * d.seq_k * 64,
                        bytes_moved=_nbytes(ins["Q"], ins["K"], ins["V"], outs["Output"]), kind="attention")


@op_implementation(op="FusedAttentionGrad", name=IMPL)
class HipFusedAttentionGrad(ONNXForward):
    """Backward of FusedAttention: what DefaultEinsumBackward and DefaultSoftmaxBackward
    (autodiff/implementations/onnx_ops.py:25-138, 237-275) compute for the chain, recomputing the
    probabilities from Q, K and the stored log-sum-exp."""
    @staticmethod
    def _pairs(node, ins, outs):
        fwd = [(ins["Q"], node.q_perm), (ins["K"], node.k_perm), (ins["V"], node.v_perm), (ins["O"], node.o_perm)]
        grad = [(outs["dQ"], node.q_perm), (outs["dK"], node.k_perm), (outs["dV"], node.v_perm), (ins["dO"], node.o_perm)]
        return fwd, grad

    @staticmethod
    def forward_can_be_applied(node, state, sdfg) -> bool:
        try:
            ins, outs = _descs(node, state, sdfg)
            fwd, grad = HipFusedAttentionGrad._pairs(node, ins, outs)
            lse = ins["LogSumExp"]
            if "Mask" in ins and attention_mask_strides(ins["Mask"], ins["Q"], ins["K"], node.q_perm, node.k_perm) is None:
                return False
            return _attn_ok(node, fwd) and _attn_ok(node, grad) and lse.dtype == torch.float32 and lse.is_contiguous()
        except Exception:
            return False

    @staticmethod
    def forward(node, state, sdfg):
        import ctypes
        ins, outs = _descs(node, state, sdfg)
        fwd, grad = HipFusedAttentionGrad._pairs(node, ins, outs)
        d = _attn_struct(fwd, ins["Q"], ins["K"], node.scale, node.q_perm, node.k_perm)
        g = _attn_struct(grad, ins["Q"], ins["K"], node.scale, node.q_perm, node.k_perm)
        ws = L.load().dmlhip_attention_backward_workspace_bytes(ctypes.byref(d))
        if "Mask" in ins:
            ms = attention_mask_strides(ins["Mask"], ins["Q"], ins["K"], node.q_perm, node.k_perm)
            call = HipCall("dmlhip_attention_masked_backward_f16",
                           [Struct(d, "dmlhip_attention_desc"), Struct(g, "dmlhip_attention_desc"), Ptr("Q"), Ptr("K"),
                            Ptr("V"), Ptr("Mask"), I64Array(ms), Ptr("O"), Ptr("LogSumExp"), Ptr("dO"), Ptr("dQ"), Ptr("dK"),
                            Ptr("dV"), Workspace(), WorkspaceBytes(), Stream()])
        else:
            call = HipCall("dmlhip_attention_backward_f16",
                           [Struct(d, "dmlhip_attention_desc"), Struct(g, "dmlhip_attention_desc"), Ptr("Q"), Ptr("K"),
                            Ptr("V"), Ptr("O"), Ptr("LogSumExp"), Ptr("dO"), Ptr("dQ"), Ptr("dK"), Ptr("dV"), Workspace(),
                            WorkspaceBytes(), Stream()])
        bh = d.batch[0] * d.batch[1]
        return _tasklet(node, state, [call], workspace_bytes=ws, flops=8 * bh * d.seq_q * d.seq_k * 64,  # four contractions; the recomputed scores are not counted
                       
                        bytes_moved=_nbytes(ins["Q"], ins["K"], ins["V"], ins["O"], ins["dO"], outs["dQ"], outs["dK"],
                                            outs["dV"]), kind="attention_backward")


# ----------------------------------------------------------------------------- several ReduceSum nodes at once
@op_implementation(op="MultiReduceSum", name=IMPL)
class HipMultiReduceSum(ONNXForward):
    """reduced__i = np.sum(data__i, axis=all but the last) (ReduceSum, pure_implementations.py:294-306, keepdims 0)
    for up to eight tensors in one pair of launches."""
    @staticmethod
    def _pairs(node, state, sdfg):
        ins, outs = _descs(node, state, sdfg)
        n = len(ins)
        return [(ins["data__%d" % i], outs["reduced__%d" % i]) for i in range(n)]

    @staticmethod
    def forward_can_be_applied(node, state, sdfg) -> bool:
        try:
            pairs = HipMultiReduceSum._pairs(node, state, sdfg)
            if not 1 <= len(pairs) <= L.MULTI_MAX:
                return False
            dt, odt = pairs[0][0].dtype, pairs[0][1].dtype
            vec = 8 if dt == torch.float16 else 4
            for x, y in pairs:
                if x.dtype != dt or y.dtype != odt or dt not in FLOAT_DTYPES or odt not in FLOAT_DTYPES:
                    return False
                if not (x.is_contiguous() and y.is_contiguous()) or len(x.shape) < 1:
                    return False
                if y.total_size != x.shape[-1] or x.shape[-1] % vec:
                    return False
            return True
        except Exception:
            return False

    @staticmethod
    def forward(node, state, sdfg):
        import ctypes
        pairs = HipMultiReduceSum._pairs(node, state, sdfg)
        n = len(pairs)
        rows = tuple(_prod(x.shape[:-1]) for x, _ in pairs)
        cols = tuple(int(x.shape[-1]) for x, _ in pairs)
        r_arr, c_arr = (ctypes.c_int64 * n)(*rows), (ctypes.c_int64 * n)(*cols)
        ws = L.load().dmlhip_reduce_sum_multi_workspace_bytes(n, r_arr, c_arr)
        call = HipCall("dmlhip_reduce_sum_multi_" + _SFX[pairs[0][0].dtype],
                       [I32(n), PtrArray(tuple("data__%d" % i for i in range(n))),
                        PtrArray(tuple("reduced__%d" % i for i in range(n))), I32(_CODE[pairs[0][1].dtype]),
                        I64Array(rows), I64Array(cols), Workspace(), WorkspaceBytes(), Stream()])
        return _tasklet(node, state, [call], workspace_bytes=ws,
                        bytes_moved=sum(_nbytes(x, y) for x, y in pairs), kind="reduce")


# ----------------------------------------------------------------------------- several equal contractions at once
@op_implementation(op="GroupedEinsum", name=IMPL)
class HipGroupedEinsum(ONNXForward):
    """Up to four PureEinsum contractions (pure_implementations.py:219-252) of identical equation, shapes and
    strides in one grouped GEMM launch — the effect HorizontalEinsumFusion (transformation/einsum_fusion.py:102-151)
    has on the Q/K/V projections, without requiring the operands to be adjacent in memory."""
    @staticmethod
    def _groups(node, state, sdfg):
        ins, outs = _descs(node, state, sdfg)
        n = len([k for k in outs if k.startswith("Output__")])
        a = [ins["A__%d" % i] for i in range(n)]
        b = [ins["B__%d" % i] for i in range(n)]
        bias = [ins["Bias__%d" % i] for i in range(n)] if "Bias__0" in ins else None
        out = [outs["Output__%d" % i] for i in range(n)]
        return n, a, b, bias, out

    @staticmethod
    def _sums(node, state, sdfg, n):
        _, outs = _descs(node, state, sdfg)
        if "InputSum__0" not in outs:
            return None
        return [outs["InputSum__%d" % i] for i in range(n)]

    @staticmethod
    def forward_can_be_applied(node, state, sdfg) -> bool:
        try:
            n, a, b, bias, out = HipGroupedEinsum._groups(node, state, sdfg)
            if not 2 <= n <= L.GROUP_MAX or a[0].dtype != torch.float16:
                return False
            eq = node.equation.replace(" ", "")
            for i in range(n):
                if (a[i].shape, a[i].strides, a[i].dtype) != (a[0].shape, a[0].strides, a[0].dtype):
                    return False
                if (b[i].shape, b[i].strides, b[i].dtype) != (b[0].shape, b[0].strides, a[0].dtype):
                    return False
                if (out[i].shape, out[i].dtype) != (out[0].shape, out[0].dtype):
                    return False
                if not _einsum_can_apply(eq, [a[i], b[i]], out[i], allow_f32_out=True):
                    return False
            plan = _einsum_plan(eq, a[0], b[0])
            if plan is None or plan.batch[0] != 1:
                return False
            if bias is not None:
                for t in bias:
                    if not (t.dtype == bias[0].dtype and t.dtype in FLOAT_DTYPES and t.is_contiguous()
                            and t.total_size == plan.n and t.shape[-1] == plan.n):
                        return False
            sums = HipGroupedEinsum._sums(node, state, sdfg, n)
            if sums is not None:
                if bias is not None or any(t.dtype != sums[0].dtype for t in sums):
                    return False
                if not all(_input_sum_ok(plan, a[i], sums[i]) for i in range(n)):
                    return False
            return True
        except Exception:
            return False

    @staticmethod
    def forward(node, state, sdfg):
        import ctypes
        n, a, b, bias, out = HipGroupedEinsum._groups(node, state, sdfg)
        eq = node.equation.replace(" ", "")
        sums = HipGroupedEinsum._sums(node, state, sdfg, n)
        if sums is not None:
            rng_ = range(n)
            return _asum_tasklet(node, state, eq, node.alpha, a, b, out, sums[0], ["A__%d" % i for i in rng_],
                                 ["B__%d" % i for i in rng_], ["Output__%d" % i for i in rng_],
                                 ["InputSum__%d" % i for i in rng_])
        plan = C.plan_contraction(eq, a[0].shape, a[0].strides, b[0].shape, b[0].strides)
        desc = _gemm_struct(plan, node.alpha, 0.0, out[0].dtype, bias[0].dtype if bias else out[0].dtype, L.ACT_NONE)
        xa, xb = ("B", "A") if plan.swapped else ("A", "B")
        ws = L.load().dmlhip_gemm_f16_workspace_bytes(ctypes.byref(desc))
        call = HipCall("dmlhip_gemm_f16_grouped",
                       [Struct(desc, "dmlhip_gemm_desc"), I32(n), PtrArray(tuple("%s__%d" % (xa, i) for i in range(n))),
                        PtrArray(tuple("%s__%d" % (xb, i) for i in range(n))),
                        PtrArray(tuple("Output__%d" % i for i in range(n))),
                        PtrArray(tuple("Bias__%d" % i for i in range(n))) if bias else Null(), Workspace(),
                        WorkspaceBytes(), Stream()])
        extra = bias or []
        return _tasklet(node, state, [call], workspace_bytes=ws, flops=plan.flops * n,
                        bytes_moved=sum(_nbytes(a[i], b[i], out[i]) for i in range(n)) + _nbytes(*extra), kind="gemm")


@op_implementation(op="EinsumSum", name=IMPL)
class HipEinsumSum(ONNXForward):
    """Sum of up to four PureEinsum contractions (pure_implementations.py:219-252) of identical equation, shapes and
    strides, optionally plus a residual of the output's shape: the ONNXSum with which autodiff accumulates gradient
    contributions (autodiff/backward_pass_generator.py:715-752) folded into the contractions that produce them.
    The operand pairs are concatenated along K in one launch; the accumulation stays in fp32."""
    @staticmethod
    def _pairs(node, state, sdfg):
        ins, outs = _descs(node, state, sdfg)
        n = len([k for k in ins if k.startswith("A__")])
        return n, [ins["A__%d" % i] for i in range(n)], [ins["B__%d" % i] for i in range(n)], ins.get("Residual"), \
            outs["Output"]

    @staticmethod
    def forward_can_be_applied(node, state, sdfg) -> bool:
        try:
            n, a, b, res, out = HipEinsumSum._pairs(node, state, sdfg)
            if not 1 <= n <= L.GROUP_MAX or a[0].dtype != torch.float16:
                return False
            eq = node.equation.replace(" ", "")
            for i in range(n):
                if (a[i].shape, a[i].strides, a[i].dtype) != (a[0].shape, a[0].strides, a[0].dtype):
                    return False
                if (b[i].shape, b[i].strides, b[i].dtype) != (b[0].shape, b[0].strides, a[0].dtype):
                    return False
                if not _einsum_can_apply(eq, [a[i], b[i]], out, allow_f32_out=True):
                    return False
            if res is not None and not (res.shape == out.shape and res.dtype == out.dtype and res.strides == out.strides):
                return False
            return _einsum_plan(eq, a[0], b[0]) is not None
        except Exception:
            return False

    @staticmethod
    def forward(node, state, sdfg):
        n, a, b, res, out = HipEinsumSum._pairs(node, state, sdfg)
        eq = node.equation.replace(" ", "")
        plan = C.plan_contraction(eq, a[0].shape, a[0].strides, b[0].shape, b[0].strides)
        desc = _gemm_struct(plan, node.alpha, 0.0, out.dtype, out.dtype, L.ACT_NONE)
        xa, xb = ("B", "A") if plan.swapped else ("A", "B")
        call = HipCall("dmlhip_gemm_f16_ksum",
                       [Struct(desc, "dmlhip_gemm_desc"), I32(n), PtrArray(tuple("%s__%d" % (xa, i) for i in range(n))),
                        PtrArray(tuple("%s__%d" % (xb, i) for i in range(n))), Ptr("Output"), Null(),
                        Ptr("Residual") if res is not None else Null(), Stream()])
        extra = [res] if res is not None else []
        return _tasklet(node, state, [call], flops=plan.flops * n,
                        bytes_moved=sum(_nbytes(a[i], b[i]) for i in range(n)) + _nbytes(out, *extra), kind="gemm")


@op_implementation(op="ScaledExpand", name=IMPL)
class HipScaledExpand(ONNXForward):
    """Broadcast X along its size-1 dims to Y's shape and multiply by a one-element Scale: what ReverseReduce
    (daceml/autodiff/implementations/dace_nodes.py:13-105) does for a Sum reduction, times the 1/n of a mean —
    one pass of the broadcasting elementwise kernel."""
    @staticmethod
    def forward_can_be_applied(node, state, sdfg) -> bool:
        try:
            ins, outs = _descs(node, state, sdfg)
            x, sc, y = ins["X"], ins["Scale"], outs["Y"]
            xs = HipScaledExpand._x_shape(node, x)
            return (_float_ok(x, sc, y) and x.dtype == y.dtype == sc.dtype and sc.total_size == 1 and y.is_contiguous()
                    and x.is_contiguous() and _prod(xs) == x.total_size and len(xs) == len(y.shape) <= L.MAX_DIMS
                    and all(a == b or a == 1 for a, b in zip(xs, y.shape)))
        except Exception:
            return False

    @staticmethod
    def _x_shape(node, x):
        return tuple(int(d) for d in node.x_shape) if node.x_shape is not None else tuple(x.shape)

    @staticmethod
    def forward(node, state, sdfg):
        ins, outs = _descs(node, state, sdfg)
        x, y = ins["X"], outs["Y"]
        shape = tuple(y.shape)
        xs = HipScaledExpand._x_shape(node, x)
        dense = C.contiguous_strides(xs)
        x_strides = tuple(0 if e == 1 else s for e, s in zip(xs, dense))
        call = HipCall("dmlhip_binary_" + _SFX[y.dtype],
                       [I32(L.MUL), Ptr("X"), Ptr("Scale"), Ptr("Y"), I32(len(shape)), I64Array(shape),
                        I64Array(x_strides), I64Array((0, ) * len(shape)), Stream()])
        return _tasklet(node, state, [call], bytes_moved=_nbytes(x, y), kind="elementwise")
