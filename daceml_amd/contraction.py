"""Einsum front end: turn an einsum equation plus operand layouts into one strided, batched GEMM.

This is host-side planning only (no device work), the counterpart of what the reference gets from
DaCe's ``create_einsum_sdfg`` when PureEinsum lowers a contraction to a BLAS library node
(daceml/onnx/op_implementations/pure_implementations.py:219-252). Operand strides are taken as they
are, so a Transpose feeding a contraction is absorbed into the GEMM's operand layout (the effect of
HorizontalEinsumFusion, daceml/transformation/einsum_fusion.py:102-151) instead of being executed.
"""
import dataclasses
from typing import Dict, List, Optional, Sequence, Tuple


class NotApplicable(Exception):
    """The equation / layout is outside what one GEMM launch covers."""


@dataclasses.dataclass
class GemmPlan:
    m: int
    n: int
    k: int
    batch: List[int]                 # three extents (1-padded)
    a_stride_m: int
    a_stride_k: int
    a_stride_batch: List[int]
    b_stride_k: int
    b_stride_n: int
    b_stride_batch: List[int]
    c_stride_m: int
    c_stride_batch: List[int]
    swapped: bool                    # operands exchanged so that the GEMM's n runs along C's last dim
    out_shape: Tuple[int, ...]

    @property
    def flops(self) -> int:
        b = 1
        for e in self.batch:
            b *= e
        return 2 * b * self.m * self.n * self.k


def parse(equation: str) -> Tuple[List[str], str]:
    eq = equation.replace(" ", "")
    if "..." in eq:
        raise NotApplicable("ellipsis not supported (as in PureEinsum.forward_can_be_applied)")
    if "->" not in eq:
        raise NotApplicable("implicit-output equations are not supported")
    lhs, rhs = eq.split("->")
    inputs = lhs.split(",")
    for term in inputs + [rhs]:
        if not term.isalpha() and term != "":
            raise NotApplicable("malformed equation %r" % equation)
        if len(set(term)) != len(term):
            raise NotApplicable("repeated index inside one operand (%r)" % term)
    return inputs, rhs


def contiguous_strides(shape: Sequence[int]) -> List[int]:
    strides, s = [], 1
    for ext in reversed(shape):
        strides.append(s)
        s *= ext
    return list(reversed(strides))


def output_shape(equation: str, shapes: Sequence[Sequence[int]]) -> Tuple[int, ...]:
    inputs, out = parse(equation)
    if len(inputs) != len(shapes):
        raise ValueError("equation has %d operands, %d shapes given" % (len(inputs), len(shapes)))
    ext: Dict[str, int] = {}
    for term, shp in zip(inputs, shapes):
        if len(term) != len(shp):
            raise ValueError("operand %r has rank %d, shape %s" % (term, len(term), tuple(shp)))
        for l, e in zip(term, shp):
            if ext.setdefault(l, e) != e:
                raise ValueError("extent mismatch for index %r" % l)
    for l in out:
        if l not in ext:
            raise ValueError("output index %r missing from the inputs" % l)
    return tuple(ext[l] for l in out)


def transpose_perm(equation: str) -> Optional[List[int]]:
    """For a one-operand equation that only permutes (``zyxw->zxyw``) return the permutation
    (EinsumTranspose, pure_implementations.py:746-778); None otherwise."""
    inputs, out = parse(equation)
    if len(inputs) != 1 or sorted(inputs[0]) != sorted(out):
        return None
    return [inputs[0].index(l) for l in out]


def _merge(letters: List[str], ext: Dict[str, int], stride_maps: List[Dict[str, int]]):
    """Merge `letters` (outer -> inner) into one (extent, strides per tensor) if every tensor lays
    them out as one strided run; None if not."""
    letters = [l for l in letters if ext[l] != 1]
    if not letters:
        return 1, [0 for _ in stride_maps]
    for sm in stride_maps:
        for outer, inner in zip(letters, letters[1:]):
            if sm[outer] != sm[inner] * ext[inner]:
                return None
    total = 1
    for l in letters:
        total *= ext[l]
    return total, [sm[letters[-1]] for sm in stride_maps]


def plan_contraction(equation: str, a_shape, a_strides, b_shape, b_strides) -> GemmPlan:
    """Plan ``equation`` (two operands) as one GEMM; the output is dense row-major.

    Raises NotApplicable when the index structure needs more than one launch (an index summed inside a
    single operand, index groups that no single stride describes, more than three batch dims, ...).
    """
    inputs, out = parse(equation)
    if len(inputs) != 2:
        raise NotApplicable("a contraction plan needs exactly two operands")
    ta, tb = inputs
    oshape = output_shape(equation, [a_shape, b_shape])
    ext: Dict[str, int] = {}
    for term, shp in ((ta, a_shape), (tb, b_shape)):
        for l, e in zip(term, shp):
            ext[l] = int(e)
    sa = {l: int(s) for l, s in zip(ta, a_strides)}
    sb = {l: int(s) for l, s in zip(tb, b_strides)}
    sc = {l: int(s) for l, s in zip(out, contiguous_strides(oshape))}

    batch = [l for l in out if l in ta and l in tb]
    m_let = [l for l in out if l in ta and l not in tb]
    n_let = [l for l in out if l in tb and l not in ta]
    k_let = [l for l in ta if l in tb and l not in out]
    lonely = [l for l in ta + tb if l not in out and not (l in ta and l in tb)]
    if lonely:
        raise NotApplicable("index %r is summed inside a single operand" % lonely[0])

    # the GEMM writes n with unit stride: the innermost non-trivial output index decides which
    # operand plays B
    inner = [l for l in out if ext[l] != 1]
    swapped = False
    if inner and inner[-1] in m_let:
        swapped = True
        ta, tb, sa, sb, m_let, n_let = tb, ta, sb, sa, n_let, m_let
    elif inner and inner[-1] in batch:
        raise NotApplicable("a batch index is innermost in the output")

    mm = _merge(m_let, ext, [sa, sc])
    nn = _merge(n_let, ext, [sb, sc])
    kk = _merge(k_let, ext, [sa, sb])
    if kk is None:  # try the other operand's order
        kk = _merge([l for l in tb if l in k_let], ext, [sa, sb])
    if mm is None or nn is None or kk is None:
        raise NotApplicable("an index group is not one strided run in some operand")
    m, (a_sm, c_sm) = mm
    n, (b_sn, c_sn) = nn
    k, (a_sk, b_sk) = kk
    if n != 1 and c_sn != 1:
        raise NotApplicable("the n indices are not innermost in the output")
    if m != 1 and n != 1 and c_sm < n:
        raise NotApplicable("m and n indices interleave in the output")

    # batch: greedily merge adjacent letters, at most three dims survive
    groups: List[List[str]] = []
    for l in batch:
        if ext[l] == 1:
            continue
        if groups and _merge(groups[-1] + [l], ext, [sa, sb, sc]) is not None:
            groups[-1].append(l)
        else:
            groups.append([l])
    if len(groups) > 3:
        raise NotApplicable("more than three independent batch dims")
    bext, bsa, bsb, bsc = [], [], [], []
    for g in groups:
        e, (x, y, z) = _merge(g, ext, [sa, sb, sc])
        bext.append(e); bsa.append(x); bsb.append(y); bsc.append(z)
    while len(bext) < 3:
        bext.insert(0, 1); bsa.insert(0, 0); bsb.insert(0, 0); bsc.insert(0, 0)

    return GemmPlan(m=m, n=n, k=k, batch=bext, a_stride_m=a_sm, a_stride_k=a_sk, a_stride_batch=bsa,
                    b_stride_k=b_sk, b_stride_n=b_sn, b_stride_batch=bsb, c_stride_m=c_sm if m != 1 else max(n, 1),
                    c_stride_batch=bsc, swapped=swapped, out_shape=oshape)


def matmul_equation(a_rank: int, b_rank: int) -> str:
    """Equation PureMatMul lowers ``MatMul(A, B)`` to (pure_implementations.py:132-191): the last two
    dims are ``ik,kj->ij``; batch letters are taken from the end of ``z..a`` minus ``i j k`` (so the
    first one is ``a``), assigned right-aligned; a dim present in one operand only appears in that
    operand and the result."""
    if a_rank < 2 or b_rank < 2:
        raise NotApplicable("1-D MatMul operands are refused (pure_implementations.py:114-121)")
    letters = [chr(ord('z') - i) for i in range(26) if chr(ord('z') - i) not in 'ijk']
    arg1, arg2, res = 'ik', 'kj', 'ij'
    na, nb = a_rank - 2, b_rank - 2
    for d in range(max(na, nb)):
        letter = letters.pop()
        if d < na:
            arg1 = letter + arg1
        if d < nb:
            arg2 = letter + arg2
        res = letter + res
    return "%s,%s->%s" % (arg1, arg2, res)


def reverse_equation(equation: str, input_idx: int) -> Tuple[List[int], str]:
    """Equation of the gradient w.r.t. input `input_idx`
    (reverse_einsum_wrt_input, daceml/autodiff/implementations/onnx_ops.py:25-51): operands are the
    output gradient followed by the other forward inputs; result is the differentiated input."""
    inputs, out = parse(equation)
    others = [i for i in range(len(inputs)) if i != input_idx]
    terms = [out] + [inputs[i] for i in others]
    return others, "%s->%s" % (",".join(terms), inputs[input_idx])
