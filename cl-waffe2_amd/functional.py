"""User-level tensor functions, decomposed into nodes the way cl-waffe2 does.

Eager mirror of ``source/base-impl`` (``!add`` ... ``!matmul``), ``!sum`` /
``!mean`` (``base-impl/reduction.lisp``) and the ``source/nn`` recipes used by a
transformer block.  Each function issues the same node sequence the reference
builds lazily and runs through ``proceed``; the nodes land on whatever device
``nodes.USING_BACKEND`` selects.

Naming: ``!add`` -> ``add``, ``A+=B`` -> ``add_``, ``!loge`` -> ``loge``,
``->contiguous`` -> ``to_contiguous``.
"""
from __future__ import annotations

import builtins as _builtins
import math
from typing import Sequence

import numpy as np

from . import lib as _lib
from . import nodes
from .tensor import HIPTensor

Number = (int, float, np.integer, np.floating)


# ---------------------------------------------------------------------------
# construction / movement
# ---------------------------------------------------------------------------

def make_tensor(shape: Sequence[int], initial_element: float = 0.0, dtype: str = "float") -> HIPTensor:
    """``(make-tensor shape :initial-element x :dtype dtype)``"""
    return HIPTensor(shape, initial_element=initial_element, dtype=dtype)


def from_numpy(a, dtype: str = "float") -> HIPTensor:
    return HIPTensor.from_numpy(a, dtype=dtype)


def move_(dst: HIPTensor, src: HIPTensor) -> HIPTensor:
    """``(!move dst src)``: MoveTensorNode, ``dst <- src``
    (``base-impl/fundamental.lisp:9-43,80-120``)."""
    return nodes.forward("MoveTensorNode", dst, src)


def copy(x: HIPTensor) -> HIPTensor:
    """``(!copy x)``: a fresh contiguous tensor of x's visible shape filled by
    MoveTensorNode (``fundamental.lisp:122-163``)."""
    return move_(HIPTensor(x.shape, initial_element=None, dtype=x.dtype), x)


def to_contiguous(x: HIPTensor) -> HIPTensor:
    """``(->contiguous x)`` (``fundamental.lisp:1059-1107``): copies only when
    the tensor is viewed, permuted or broadcast."""
    return x if x.is_contiguous() else copy(x)


def view(x: HIPTensor, *subscripts) -> HIPTensor:
    return x.view(*subscripts)


def permute(x: HIPTensor, *order: int) -> HIPTensor:
    return x.permute(*order)


def reshape(x: HIPTensor, *shape: int) -> HIPTensor:
    """``(!reshape x ...)`` (``fundamental.lisp:273-350``): same storage, new
    shape; a non-contiguous source is materialised first.  One extent may be
    -1."""
    shape = list(shape)
    if shape.count(-1) == 1:
        known = math.prod(s for s in shape if s != -1)
        shape[shape.index(-1)] = x.size // _builtins.max(known, 1)
    if math.prod(shape) != x.size:
        raise ValueError(f"reshape: cannot reshape {x.shape} into {shape}")
    src = to_contiguous(x)
    return HIPTensor(shape, vec=src.vec, dtype=src.dtype)


class Transposed:
    """Marker returned by ``t``: the last two axes are swapped lazily and the
    flag is consumed by ``matmul`` (``LazyTransposeNode``,
    ``base-impl/matrix-ops.lisp:34-78``)."""

    def __init__(self, tensor: HIPTensor):
        self.tensor = tensor

    @property
    def shape(self):
        s = self.tensor.shape
        return s[:-2] + [s[-1], s[-2]]


def t(x: HIPTensor) -> Transposed:
    """``(!t x)``"""
    return Transposed(x)


# ---------------------------------------------------------------------------
# broadcasting helpers
# ---------------------------------------------------------------------------

def scalar_tensor(value: float, like: HIPTensor) -> HIPTensor:
    """A ``(1 ... 1)`` tensor viewed ``(:broadcast n)`` on every axis, which is
    how ``!scalar-add`` & co. feed a scalar to a tensor node
    (``base-impl/arithmetic.lisp:31-51,216-262``)."""
    s = HIPTensor([1] * like.ndim, initial_element=value if like.dtype != "float" else float(value),
                  dtype=like.dtype)
    return s.view(*[(":broadcast", n) if n != 1 else True for n in like.shape])


def flexible(y: HIPTensor, like: HIPTensor) -> HIPTensor:
    """Rank-extend ``y`` on the left and broadcast its size-1 axes against
    ``like`` (what ``!flexible`` + the automatic broadcast of ``forward
    :around`` do, ``vm/nodes/node.lisp:171-182``, ``broadcast.lisp:22``)."""
    ys, ls = y.shape, like.shape
    if ys == ls:
        return y
    if len(ys) > len(ls):
        raise ValueError(f"cannot broadcast {ys} to {ls}")
    if len(ys) < len(ls):
        if not y.is_contiguous():
            y = copy(y)
        y = HIPTensor([1] * (len(ls) - len(ys)) + ys, vec=y.vec, dtype=y.dtype)
        ys = y.shape
    subs = []
    for a, b in zip(ys, ls):
        if a == b:
            subs.append(True)
        elif a == 1:
            subs.append((":broadcast", b))
        else:
            raise ValueError(f"cannot broadcast {ys} to {ls}")
    # T would reset an existing slice; only touch axes that need broadcasting
    if all(s is True for s in subs):
        return y
    views = list(y.views)
    from .tensor import parse_view
    for i, s in enumerate(subs):
        if s is not True:
            views[i] = parse_view(y.orig_shape[i], y.views[i], s)
    return HIPTensor(y.orig_shape, vec=y.vec, strides=y.stride, views=views, offset=y.initial_offset,
                     dtype=y.dtype)


def _operand(y, like: HIPTensor) -> HIPTensor:
    if isinstance(y, Number):
        return scalar_tensor(y, like)
    return flexible(y, like)


# ---------------------------------------------------------------------------
# arithmetic
# ---------------------------------------------------------------------------

def add_(x: HIPTensor, y) -> HIPTensor:
    """``(A+=B x y)``: AddNode in place in x."""
    return nodes.forward("AddNode", x, _operand(y, x))


def sub_(x: HIPTensor, y) -> HIPTensor:
    return nodes.forward("SubNode", x, _operand(y, x))


def mul_(x: HIPTensor, y) -> HIPTensor:
    return nodes.forward("MulNode", x, _operand(y, x))


def div_(x: HIPTensor, y) -> HIPTensor:
    return nodes.forward("DivNode", x, _operand(y, x))


def _out_of_place(node: str, x, y) -> HIPTensor:
    """``!add``-family (``base-impl/arithmetic.lisp:114-177,367-434``): the left
    operand is copied, the node runs in place on the copy."""
    if isinstance(x, Number):
        # scalar op tensor: s + T, s * T commute; s - T = s + (-1 * T);
        # s / T = s * (1 / T)   (arithmetic.lisp:180-209,407-434)
        if node == "AddNode":
            return add_(copy(y), x)
        if node == "MulNode":
            return mul_(copy(y), x)
        if node == "SubNode":
            return add_(mul_(copy(y), -1.0), x)
        return mul_(reciprocal(y), x)
    if isinstance(y, Number):
        return nodes.forward(node, copy(x), scalar_tensor(y, x))
    if x.shape == y.shape:
        return nodes.forward(node, copy(x), y)
    out_shape = list(np.broadcast_shapes(tuple(x.shape), tuple(y.shape)))
    if x.shape == out_shape:
        left = copy(x)
    else:  # x is the smaller operand: expand it into a full-size tensor first
        left = move_(HIPTensor(out_shape, initial_element=None, dtype=x.dtype), flexible(x, _ShapeOnly(out_shape)))
    return nodes.forward(node, left, flexible(y, left))


def add(x, y) -> HIPTensor:
    return _out_of_place("AddNode", x, y)


def sub(x, y) -> HIPTensor:
    return _out_of_place("SubNode", x, y)


def mul(x, y) -> HIPTensor:
    return _out_of_place("MulNode", x, y)


def div(x, y) -> HIPTensor:
    return _out_of_place("DivNode", x, y)


def reciprocal(x: HIPTensor) -> HIPTensor:
    """``(!reciprocal x)`` = DivNode(ones, x) (``arithmetic.lisp:180-209``)."""
    return nodes.forward("DivNode", HIPTensor(x.shape, initial_element=1.0), x)


# ---------------------------------------------------------------------------
# mathematics
# ---------------------------------------------------------------------------

def _math(node: str, x: HIPTensor, out: HIPTensor | None = None) -> HIPTensor:
    """``(!exp x :-> out)``: ``out`` defaults to a fresh tensor (the pruned
    ``(!copy x :maybe-in-place t)`` of ``base-impl/mathematics.lisp:13-120``)."""
    if out is None:
        out = HIPTensor(x.shape, initial_element=None, dtype=x.dtype)
    return nodes.forward(node, x, out)


def sin(x, out=None): return _math("SinNode", x, out)
def cos(x, out=None): return _math("CosNode", x, out)
def tanh(x, out=None): return _math("TanhNode", x, out)
def exp(x, out=None): return _math("ExpNode", x, out)
def loge(x, out=None): return _math("LogENode", x, out)
def sqrt(x, out=None): return _math("SqrtNode", x, out)
def abs(x, out=None): return _math("AbsNode", x, out)  # noqa: A001 - mirrors !abs
def tan(x, out=None): return _math("TanNode", x, out)
def asin(x, out=None): return _math("ASinNode", x, out)
def acos(x, out=None): return _math("ACosNode", x, out)
def atan(x, out=None): return _math("ATanNode", x, out)
def sinh(x, out=None): return _math("SinHNode", x, out)
def cosh(x, out=None): return _math("CosHNode", x, out)
def log2(x, out=None): return _math("Log2Node", x, out)
def log10(x, out=None): return _math("Log10Node", x, out)
def log1p(x, out=None): return _math("Log1pNode", x, out)
def sign(x, out=None): return _math("SignNode", x, out)
def square(x, out=None): return _math("SquareNode", x, out)
def asinh(x, out=None): return _math("ASinHNode", x, out)
def acosh(x, out=None): return _math("ACosHNode", x, out)
def atanh(x, out=None): return _math("ATanHNode", x, out)


def expt(x: HIPTensor, n: float, out: HIPTensor | None = None) -> HIPTensor:
    """``(!expt x n)`` (``mathematics.lisp:267-303``)."""
    if out is None:
        out = HIPTensor(x.shape, initial_element=None, dtype=x.dtype)
    return nodes.forward("ExptNode", x, out, float(n))


# ---------------------------------------------------------------------------
# padding / unfold (source/base-impl/utils.lisp:4-140, source/nn/im2col.lisp)
# ---------------------------------------------------------------------------

def padding(x: HIPTensor, pad_width) -> HIPTensor:
    """``(padding tensor pad-width)``: a zero tensor of the padded shape, a view of
    its interior, ``x`` moved into the view.  ``pad_width`` holds ``(before,
    after)`` per axis, or ``True`` for an axis left alone."""
    if len(pad_width) != len(x.shape):
        raise ValueError("padding: one (before, after) pair or True per axis")
    widths = [(0, 0) if w is True else (int(w[0]), int(w[1])) for w in pad_width]
    if all(w == (0, 0) for w in widths):
        return x
    out = HIPTensor([n + b + a for n, (b, a) in zip(x.shape, widths)])
    inner = out.view(*[True if w == (0, 0) else (w[0], w[0] + n) for n, w in zip(x.shape, widths)])
    move_(inner, x)
    return out


def conv_out_size(size: int, pad: int, dilation: int, kernel: int, stride: int) -> int:
    """``conv-out-size`` (``source/nn/pool.lisp:10-17``)."""
    return (size + 2 * pad - dilation * (kernel - 1) - 1) // stride + 1


def im2col(padded_x: HIPTensor, kernel_size, h_out: int, w_out: int, stride, pad, dilation) -> HIPTensor:
    """``!im2col`` (``source/nn/im2col.lisp:15-49``): Im2ColNode into a fresh
    ``[N C k-h k-w h-out w-out]`` tensor, then permuted to (N h-out w-out C k-h k-w)
    and reshaped to ``[(N h-out w-out) (C k-h k-w)]``."""
    N, Cc = padded_x.shape[:2]
    col = HIPTensor([N, Cc, kernel_size[0], kernel_size[1], h_out, w_out])
    nodes.forward("Im2ColNode", to_contiguous(padded_x), col, stride, pad, dilation)
    return reshape(col.permute(0, 4, 5, 1, 2, 3), N * h_out * w_out, Cc * kernel_size[0] * kernel_size[1])


def unfold_composed(x: HIPTensor, dilation, kernel_size, stride, pad) -> HIPTensor:
    """``(unfold input dilation kernel-size stride padding)``
    (``source/nn/im2col.lisp:51-95``) node for node: sliding local blocks of a
    ``[N C H W]`` tensor as rows of a ``[(N h-out w-out) (C k-h k-w)]`` matrix.  The
    input is padded by ``(pad, pad + out mod stride)`` on each spatial axis first, as
    the reference does."""
    if len(x.shape) != 4:
        raise ValueError("unfold takes a [N C H W] tensor")
    H, W = x.shape[2:]
    h_out = conv_out_size(H, pad[0], dilation[0], kernel_size[0], stride[0])
    w_out = conv_out_size(W, pad[1], dilation[0], kernel_size[1], stride[1])   # (car dilation) twice: sic
    px = padding(x, [True, True, (pad[0], pad[0] + h_out % stride[0]), (pad[1], pad[1] + w_out % stride[1])])
    return im2col(px, kernel_size, h_out, w_out, stride, pad, dilation)


def unfold(x: HIPTensor, dilation, kernel_size, stride, pad) -> HIPTensor:
    """``(unfold input dilation kernel-size stride padding)``.  On :float tensors with
    dilation 1 and the symbolic path enabled this is ONE node (HIP-Unfold-Node, the
    bypass ``unfold-hip`` of the Lisp glue), bit for bit the matrix the composition
    leaves (`unfold_composed`); otherwise the composition itself."""
    if len(x.shape) != 4:
        raise ValueError("unfold takes a [N C H W] tensor")
    if not (ENABLE_SYMBOLIC_PATH and x.dtype == "float" and tuple(dilation) == (1, 1)):
        return unfold_composed(x, dilation, kernel_size, stride, pad)
    N, Cc, H, W = x.shape
    h_out = conv_out_size(H, pad[0], 1, kernel_size[0], stride[0])
    w_out = conv_out_size(W, pad[1], 1, kernel_size[1], stride[1])
    out = HIPTensor([N * h_out * w_out, Cc * kernel_size[0] * kernel_size[1]], initial_element=None)
    try:
        return nodes.forward("HIP-Unfold-Node", to_contiguous(x), out, kernel_size, stride, pad)
    except _lib.HIPError as err:
        if err.code != _lib.EUNSUPPORTED:  # rows too wide for the kernel's staging memory: compose
            raise
        return unfold_composed(x, dilation, kernel_size, stride, pad)


def unfold_backward(dcol: HIPTensor, x_shape, kernel_size, stride, pad) -> HIPTensor:
    """The gradient of :func:`unfold` with respect to its input, as the reference's nodes derive it:
    the reshape and the permutation undone (a copy into ``[N C k-h k-w h-out w-out]``),
    Col2ImNode into the padded image, the interior of the padding."""
    N, Cc, H, W = x_shape
    kh, kw = kernel_size
    h_out = conv_out_size(H, pad[0], 1, kh, stride[0])
    w_out = conv_out_size(W, pad[1], 1, kw, stride[1])
    col = to_contiguous(reshape(dcol, N, h_out, w_out, Cc, kh, kw).permute(0, 3, 4, 5, 1, 2))
    Hp, Wp = H + 2 * pad[0] + h_out % stride[0], W + 2 * pad[1] + w_out % stride[1]
    px = HIPTensor([N, Cc, Hp, Wp], initial_element=None)
    nodes.forward("Col2ImNode", col, px, stride, pad, (1, 1))
    if (Hp, Wp) == (H, W):
        return px
    return to_contiguous(px.view(True, True, (pad[0], pad[0] + H), (pad[1], pad[1] + W)))


# ---------------------------------------------------------------------------
# compare / where (source/base-impl/logical.lisp)
# ---------------------------------------------------------------------------

def where(x: HIPTensor, condition: str, scal: float, true_then: float = 1.0, false_then: float = 0.0,
          out: HIPTensor | None = None) -> HIPTensor:
    """``(!where x #'(lambda (e) (condition e scal)) ...)`` for the five
    predicates with a device kernel (``logical.lisp:65-110``): ``out_i`` is
    ``true_then`` where ``x_i condition scal`` holds, else ``false_then``."""
    if out is None:
        out = HIPTensor(x.shape, initial_element=None, dtype=x.dtype)
    return nodes.forward("Where-Operation-Node", x, out, condition, float(scal), true_then, false_then)


def compare(x: HIPTensor, y: HIPTensor, condition: str, true_then: float = 1.0,
            false_then: float = 0.0, out: HIPTensor | None = None) -> HIPTensor:
    """``(!compare x y condition ...)`` (``logical.lisp:112-156``)."""
    if out is None:
        out = HIPTensor(x.shape, initial_element=None, dtype=x.dtype)
    return nodes.forward("Compare-Operation-Node", x, y, out, condition, true_then, false_then)


def _scal_cmp(condition):
    def f(a: HIPTensor, scal: float, out: HIPTensor | None = None, true_then: float = 1.0,
          false_then: float = 0.0) -> HIPTensor:
        return where(a, condition, scal, true_then, false_then, out)
    f.__doc__ = f"``(A{condition}scal A scal)`` (``logical.lisp:162-194``)."
    return f


def _mat_cmp(condition):
    def f(a: HIPTensor, b: HIPTensor, out: HIPTensor | None = None, true_then: float = 1.0,
          false_then: float = 0.0) -> HIPTensor:
        return compare(a, b, condition, true_then, false_then, out)
    f.__doc__ = f"``(A{condition}B A B)`` (``logical.lisp:196-225``)."
    return f


a_gt_scal, a_lt_scal, a_ge_scal, a_le_scal, a_eq_scal = (_scal_cmp(c) for c in (">", "<", ">=", "<=", "="))
a_gt_b, a_lt_b, a_ge_b, a_le_b, a_eq_b = (_mat_cmp(c) for c in (">", "<", ">=", "<=", "="))


def relu(x: HIPTensor) -> HIPTensor:
    """``(!relu x)`` = ``(!mul x (A>scal x 0.0))`` (``source/nn/activation.lisp:15-26``)."""
    return mul(x, a_gt_scal(x, 0.0))


def sigmoid(x: HIPTensor) -> HIPTensor:
    """``(!sigmoid x)`` = ``(!div 1 (!add 1 (!exp (!mul -1 x))))``
    (``source/nn/activation.lisp:28-43``)."""
    return div(1.0, add(1.0, exp(mul(-1.0, x))))


def leaky_relu(x: HIPTensor, negative_slope: float = 0.01) -> HIPTensor:
    """``(!leaky-relu x :negative-slope 0.01)`` = ``x * (A>=scal x 0.0 :true-then 1.0
    :false-then slope)`` (``source/nn/activation.lisp:68-92``)."""
    return mul(x, where(x, ">=", 0.0, 1.0, float(np.float32(negative_slope))))


def _fused_activation(op: int, x: HIPTensor, out: HIPTensor | None, p: float = 0.0) -> HIPTensor:
    if out is None:
        out = HIPTensor(x.shape, initial_element=None)
    return nodes.forward("HIP-Activation-Node", x, out, op, float(p))


def relu_fused(x: HIPTensor, out: HIPTensor | None = None) -> HIPTensor:
    """!relu in one kernel; bit-identical to the two-node recipe."""
    return _fused_activation(_lib.RELU, x, out)


def sigmoid_fused(x: HIPTensor, out: HIPTensor | None = None) -> HIPTensor:
    """!sigmoid in one kernel; every step rounded as its node, hence bit-identical."""
    return _fused_activation(_lib.SIGMOID, x, out)


def leaky_relu_fused(x: HIPTensor, negative_slope: float = 0.01, out: HIPTensor | None = None) -> HIPTensor:
    return _fused_activation(_lib.LEAKY_RELU, x, out, float(np.float32(negative_slope)))


# ---------------------------------------------------------------------------
# max / min / argmax / argmin (source/base-impl/matrix-ops.lisp:197-470)
# ---------------------------------------------------------------------------

def _select(node: str, x: HIPTensor, axis: int, out: HIPTensor | None, dtype: str) -> HIPTensor:
    """The reference keeps the leading ``rank - axis`` axes -- ``(butlast (shape
    tensor) axis)`` -- and reduces over everything behind them, viewed as one run:
    ``x`` is reshaped to ``(kept..., t)`` and ``out`` is ``(kept..., 1)``.  For
    the default ``axis = -1`` of a matrix that is the usual row-wise result."""
    rank = len(x.shape)
    axis = axis + rank if axis < 0 else axis
    kept = list(x.shape[:rank - axis]) if axis > 0 else list(x.shape)
    flat = reshape(x, *kept, -1)
    if out is None:
        out = HIPTensor(kept + [1], initial_element=None, dtype=dtype)
    return nodes.forward(node, flat, out)


def _keepdims(result: HIPTensor, base: HIPTensor) -> HIPTensor:
    """``keepdims`` of ``matrix-ops.lisp:385-393``: size-1 axes of the result are
    broadcast back to the extent the source has there."""
    subs = [(":broadcast", s2) if (s1 == 1 and s2 != 1) else True
            for s1, s2 in zip(result.shape, base.shape)]
    return result.view(*subs)


def max(x: HIPTensor, axis: int = -1, out: HIPTensor | None = None, keepdims: bool = False):  # noqa: A001
    """``(!max tensor :axis :out :keepdims)``."""
    r = _select("MaxValue-Node", x, axis, out, x.dtype)
    return _keepdims(r, x) if keepdims else r


def min(x: HIPTensor, axis: int = -1, out: HIPTensor | None = None, keepdims: bool = False):  # noqa: A001
    """``(!min tensor :axis :out :keepdims)``."""
    r = _select("MinValue-Node", x, axis, out, x.dtype)
    return _keepdims(r, x) if keepdims else r


def argmax(x: HIPTensor, axis: int = -1, out: HIPTensor | None = None) -> HIPTensor:
    """``(!argmax tensor :axis :out)``: a :uint32 tensor of positions within the
    reduced run."""
    return _select("ArgMax-Node", x, axis, out, "uint32")


def argmin(x: HIPTensor, axis: int = -1, out: HIPTensor | None = None) -> HIPTensor:
    """``(!argmin tensor :axis :out)``."""
    return _select("ArgMin-Node", x, axis, out, "uint32")


# ---------------------------------------------------------------------------
# reductions
# ---------------------------------------------------------------------------

def _axes(axis, ndim: int) -> list[int]:
    if axis is True:
        return list(range(ndim))
    if isinstance(axis, (int, np.integer)):
        axis = [int(axis)]
    return sorted(a + ndim if a < 0 else a for a in axis)


# Mirrors cl-waffe2/vm.nodes:*enable-symbolic-path* (vm/nodes/symbolic.lisp:118-131):
# when true, !sum / !mean on :float tensors build the one-node HIP-Sum-Node instead of
# the reference's three-node composition, as the define-bypass rules of the Lisp glue do.
ENABLE_SYMBOLIC_PATH = True


def _broadcast_view_of(out: HIPTensor, shape, axes) -> HIPTensor:
    """`out` viewed ``(:broadcast n)`` on the reduced axes (reduction.lisp:65-69); existing
    (non-broadcast) views on `out` stay intact."""
    from .tensor import parse_view
    view_args = [(":broadcast", shape[i]) if (i in axes and shape[i] != 1) else True
                 for i in range(len(shape))]
    views = list(out.views)
    for i, s in enumerate(view_args):
        if s is not True:
            views[i] = parse_view(out.orig_shape[i], out.views[i], s)
    return HIPTensor(out.orig_shape, vec=out.vec, strides=out.stride, views=views,
                     offset=out.initial_offset, dtype=out.dtype)


def sum(x: HIPTensor, axis=True, out: HIPTensor | None = None, keepdims: bool = False,  # noqa: A001
        div_by=None) -> HIPTensor:
    """``(!sum tensor :axis :-> :keepdims)``.  On :float tensors with the symbolic path
    enabled this is ONE node (HIP-Sum-Node: `out` overwritten with the sums, divided by
    ``div_by`` for !mean), whose bits equal those of the reference's composition on a
    zeroed `out`; otherwise the composition itself (`sum_composed`)."""
    if not (ENABLE_SYMBOLIC_PATH and x.dtype == "float" and (out is None or out.dtype == "float")):
        return sum_composed(x, axis=axis, out=out, keepdims=keepdims, div_by=div_by)
    axes = _axes(axis, x.ndim)
    shape = list(x.shape)
    out_shape = [1 if i in axes else n for i, n in enumerate(shape)]
    if out is None:
        out = HIPTensor(out_shape, dtype=x.dtype, initial_element=None)  # overwritten: no zero fill
    elif out.shape != out_shape:
        raise ValueError(f"!sum: the given out's shape is {out.shape}, but expected: {out_shape}")
    out_bc = _broadcast_view_of(out, shape, axes)
    nodes.forward("HIP-Sum-Node", out_bc, x, 1.0 if div_by is None else float(div_by))
    return out_bc if keepdims else out


def sum_composed(x: HIPTensor, axis=True, out: HIPTensor | None = None, keepdims: bool = False,
                 div_by=None) -> HIPTensor:
    """``(!sum tensor :axis :-> :keepdims)`` exactly as
    ``base-impl/reduction.lisp:5-79`` composes it: zero-fill ``out`` by
    multiplying with 0, view it ``(:broadcast n)`` on the reduced axes, AddNode
    ``x`` into that stride-0 view, then undo (or keep) the broadcast."""
    axes = _axes(axis, x.ndim)
    shape = list(x.shape)
    out_shape = [1 if i in axes else n for i, n in enumerate(shape)]
    if out is None:
        out = HIPTensor(out_shape, dtype=x.dtype)
    elif out.shape != out_shape:
        raise ValueError(f"!sum: the given out's shape is {out.shape}, but expected: {out_shape}")
    out = mul_(out, 0.0)  # A*=scal out 0  (reduction.lisp:63)
    out_bc = _broadcast_view_of(out, shape, axes)
    add_(out_bc, x)  # A+=B out* tensor: accumulation into a stride-0 destination
    result = out_bc if keepdims else out
    if div_by is not None:
        div_(out, float(div_by))
    return result


def mean(x: HIPTensor, axis=True, out: HIPTensor | None = None, keepdims: bool = False) -> HIPTensor:
    """``(!mean ...)`` = ``!sum`` with ``:div-by`` the number of reduced
    elements (``reduction.lisp:81-136``)."""
    n = 1
    for a in _axes(axis, x.ndim):
        n *= x.shape[a]
    return sum(x, axis=axis, out=out, keepdims=keepdims, div_by=float(n))


# ---------------------------------------------------------------------------
# matmul
# ---------------------------------------------------------------------------

def matmul(a, b, out: HIPTensor | None = None, bias: HIPTensor | None = None,
           residual: HIPTensor | None = None, activation: str | None = None,
           causal: int = 0) -> HIPTensor:
    """``(!matmul a b)`` (``base-impl/matrix-ops.lisp:80-173``): ``!t`` operands
    become transpose flags, any other non-trivial layout of the last two axes is
    materialised with ``->contiguous``, a lower-rank operand is broadcast over
    the batch axes, and the output is a fresh ``(~ i k)`` tensor.

    The keyword options fuse what would otherwise be separate nodes into the
    product's epilogue: ``act(a @ b + bias) + residual`` (``activation='gelu'``),
    ``causal=1`` when only the lower triangle of a square product is needed,
    ``causal=2`` when ``a`` is lower-triangular."""
    trans_a = isinstance(a, Transposed)
    trans_b = isinstance(b, Transposed)
    at = a.tensor if trans_a else a
    bt = b.tensor if trans_b else b

    def ready(x: HIPTensor) -> HIPTensor:
        shape, strides, _ = x.geometry()
        ok = (shape[-1] == 1 or strides[-1] == 1) and (shape[-2] == 1 or strides[-2] >= shape[-1])
        return x if ok else copy(x)

    at, bt = ready(at), ready(bt)
    ashape = a.shape if trans_a else at.shape
    bshape = b.shape if trans_b else bt.shape
    batch = ashape[:-2] if len(ashape) >= len(bshape) else bshape[:-2]
    if out is None:
        out = HIPTensor(list(batch) + [ashape[-2], bshape[-1]], dtype=at.dtype, initial_element=None)

    def with_batch(x: HIPTensor) -> HIPTensor:
        if x.shape[:-2] == list(batch):
            return x
        return flexible(x, _ShapeOnly(list(batch) + x.shape[-2:]))

    return nodes.forward("MatMulNode", with_batch(at), with_batch(bt), out,
                         trans_a=trans_a, trans_b=trans_b, bias=bias, residual=residual,
                         activation=activation, causal=causal)


class _ShapeOnly:
    def __init__(self, shape):
        self.shape = list(shape)
        self.ndim = len(shape)


# ---------------------------------------------------------------------------
# nn recipes
# ---------------------------------------------------------------------------

def softmax(x: HIPTensor, avoid_overflow: bool = True, axis=1) -> HIPTensor:
    """``(!softmax x :avoid-overflow t :axis 1)`` node for node
    (``source/nn/activation.lisp:126-159``).  Note that the reference subtracts
    the MEAN along ``axis``, not the max."""
    if avoid_overflow:
        x1 = sub(x, mean(x, axis=axis, keepdims=True))
        expx1 = exp(x1)
        z = sum(expx1, axis=axis, keepdims=True)
        return div(expx1, z)
    x1 = exp(x)
    return div(x1, sum(x1, axis=axis, keepdims=True))


def softmax_fused(x: HIPTensor, out: HIPTensor | None = None) -> HIPTensor:
    """Max-subtracted softmax over the last axis in one kernel (HIP-Softmax-Node).  A given
    ``out`` must be a contiguous :float tensor of x's shape that starts at its storage."""
    x = to_contiguous(x)
    if out is None:
        out = HIPTensor(x.shape, initial_element=None)
    return nodes.forward("HIP-Softmax-Node", x, out)


def causal_softmax_fused(scores: HIPTensor, scale: float = 1.0, out: HIPTensor | None = None) -> HIPTensor:
    """softmax over j <= i of ``scale * scores[..., i, j]``, zero above the diagonal, in one
    kernel (HIP-Causal-Softmax-Node): the scaling MulNode, the mask's AddNode and !softmax of
    causal attention."""
    scores = to_contiguous(scores)
    if out is None:
        out = HIPTensor(scores.shape, initial_element=None)
    return nodes.forward("HIP-Causal-Softmax-Node", scores, out, float(scale))


def linear(x: HIPTensor, w: HIPTensor, b: HIPTensor, activation: str | None = None,
           residual: HIPTensor | None = None, out: HIPTensor | None = None) -> HIPTensor:
    """``act(x . w + b) + residual`` for x[~ k], w[k n], b[n] as ONE node (HIP-Linear-Node /
    HIP-Linear-Residual-Node; ``!linear-hip`` of the Lisp glue): the MatMulNode, the bias's
    AddNode, !gelu and the residual's AddNode of ``examples/gpt-2/model.lisp:109-137``.
    Leading axes of x are folded into rows."""
    if activation not in (None, "gelu"):
        raise ValueError("linear: activation must be None or 'gelu'")
    if residual is not None and activation is not None:
        raise ValueError("linear: a residual closes a branch without activation")
    k, n = x.shape[-1], w.shape[-1]
    x2 = reshape(x, -1, k)
    if out is None:
        out = HIPTensor(list(x.shape[:-1]) + [n], initial_element=None)
    out2 = reshape(out, -1, n) if out.is_contiguous() else None
    if out2 is None:
        raise ValueError("linear: out must be contiguous")
    w2 = to_contiguous(w)
    if residual is not None:
        nodes.forward("HIP-Linear-Residual-Node", x2, w2, b, reshape(residual, -1, n), out2)
    else:
        nodes.forward("HIP-Linear-Node", x2, w2, b, out2, activation)
    return out


def attention(q: HIPTensor, k: HIPTensor, v: HIPTensor, out: HIPTensor | None = None,
              scale: float | None = None, causal: bool = False, lse: HIPTensor | None = None) -> HIPTensor:
    """softmax(scale q k^T [+ causal mask]) v for (batch, heads, seq, 64) views in
    one kernel (HIP-Attention-Node; ``!attention-hip`` of the Lisp glue): the fused form of
    SelfAttention's !matmul / !softmax / !matmul chain (``examples/gpt-2/utils.lisp:222-243``).
    Operands may be any views whose last axis is contiguous (heads read in
    place from a fused projection); ``out`` defaults to a fresh (B, H, T, 64)
    tensor."""
    if not (len(q.shape) == len(k.shape) == len(v.shape) == 4) or \
            not (list(q.shape) == list(k.shape) == list(v.shape)):
        raise ValueError("attention expects three (batch, heads, seq, head_dim) tensors of one shape")
    B, H, T, hd = q.shape
    if out is None:
        out = HIPTensor([B, H, T, hd], initial_element=None)
    return nodes.forward("HIP-Attention-Node", q, k, v, out, 1.0 / math.sqrt(hd) if scale is None else scale,
                         causal, lse)


def gelu(x: HIPTensor) -> HIPTensor:
    """``(!gelu x)`` node for node (``source/nn/activation.lisp:45-66``):
    0.5 x (1 + tanh(sqrt(2/pi) (x + 0.044715 x^3)))."""
    inner = add(x, mul(expt(x, 3), 0.044715))
    th = tanh(mul(inner, float(np.float32(math.sqrt(2.0 / math.pi)))))
    return mul(mul(x, 0.5), add(th, 1.0))


def gelu_fused(x: HIPTensor, out: HIPTensor | None = None) -> HIPTensor:
    """!gelu (tanh form) in one kernel (HIP-Activation-Node)."""
    return _fused_activation(_lib.GELU, x, out)


def layer_norm(x: HIPTensor, g: HIPTensor, b: HIPTensor, eps: float = 1.0e-5) -> HIPTensor:
    """``LayerNorm-Revisit`` node for node (``examples/gpt-2/utils.lisp:114-127``;
    same recipe as ``source/nn/norms.lisp:72-82``)."""
    u = mean(x, axis=-1, keepdims=True)
    xc = sub(x, u)
    s = mean(expt(xc, 2), axis=-1, keepdims=True)
    xn = div(xc, sqrt(add(to_contiguous(s), eps)))
    return add(mul(xn, g), b)


def layer_norm_fused(x: HIPTensor, g: HIPTensor, b: HIPTensor, eps: float = 1.0e-5,
                     out: HIPTensor | None = None) -> HIPTensor:
    """LayerNorm over the last axis in one kernel (HIP-LayerNorm-Node; ``!layer-norm-hip``).
    gamma, beta and a given ``out`` must be contiguous :float tensors that start at their
    storage, of shapes (cols,), (cols,) and x's."""
    x = to_contiguous(x)
    if out is None:
        out = HIPTensor(x.shape, initial_element=None)
    return nodes.forward("HIP-LayerNorm-Node", x, g, b, out, float(eps))


def layer_norm_backward(x: HIPTensor, g: HIPTensor, dout: HIPTensor, eps: float = 1.0e-5):
    """(dx, dgamma, dbeta) of LayerNorm over the last axis from the saved input: one row kernel and a
    small fold (HIP-LayerNorm-Node-backward); rows beyond 8192 columns in pieces over several workgroups.
    The node composition for the other element types."""
    cols = x.shape[-1]
    if x.dtype != "float":
        return layer_norm_backward_composed(x, g, dout, eps)
    x2, d2 = to_contiguous(x), to_contiguous(dout)
    dx = HIPTensor(list(x.shape), initial_element=None)
    dg, db = HIPTensor([cols], initial_element=None), HIPTensor([cols], initial_element=None)
    nodes.forward("HIP-LayerNorm-Node-backward", x2, g, d2, dx, dg, db, float(eps))
    return dx, dg, db


def layer_norm_backward_composed(x: HIPTensor, g: HIPTensor, dout: HIPTensor, eps: float = 1.0e-5):
    """(dx, dgamma, dbeta) of LayerNorm over the last axis, composed node for node the way
    ``layer-norm-gradients`` of the Lisp glue composes it for rows beyond the kernel's width:
    with xh = (x - u) rstd and dyh = dout g,
    dx = rstd (dyh - mean(dyh) - xh mean(dyh xh)), dgamma = sum_rows dout xh, dbeta = sum_rows dout."""
    cols = x.shape[-1]
    x2, d2 = reshape(x, -1, cols), reshape(dout, -1, cols)
    u = mean(x2, axis=-1, keepdims=True)
    xc = sub(x2, u)
    s = mean(mul(xc, xc), axis=-1, keepdims=True)
    rstd = reciprocal(sqrt(add(to_contiguous(s), eps)))
    xh = mul(xc, rstd)
    dyh = mul(d2, g)
    m1 = mean(dyh, axis=-1, keepdims=True)
    m2 = mean(mul(dyh, xh), axis=-1, keepdims=True)
    dx = mul(sub(sub(dyh, m1), mul(xh, m2)), rstd)
    dg = sum(mul(d2, xh), axis=0)
    db = sum(d2, axis=0)
    return HIPTensor(x.shape, vec=dx.vec), reshape(dg, cols), reshape(db, cols)


# ---------------------------------------------------------------------------
# backward of the fused nodes, composed the way the :backward bodies of the Lisp glue
# (lisp/fusion.lisp) compose them: the same node sequences, so the float64 checks of
# these functions are checks of those formulas
# ---------------------------------------------------------------------------

def gelu_derivative(x: HIPTensor) -> HIPTensor:
    """d/dx of 0.5 x (1 + tanh u), u = c (x + a x^3): 0.5 (1 + t) + 0.5 x (1 - t^2) c (1 + 3 a x^2),
    node for node (``gelu-derivative`` of the Lisp glue; the recipe of
    ``source/nn/activation.lisp:45-66`` differentiated).  The one-kernel form is `activation_backward`."""
    c = float(np.float32(math.sqrt(2.0 / math.pi)))
    a = 0.044715
    x2 = mul(x, x)
    u = mul(add(x, mul(mul(x2, x), a)), c)
    th = tanh(u)
    du = mul(add(mul(x2, 3 * a), 1.0), c)
    left = mul(add(th, 1.0), 0.5)
    right = mul(mul(x, 0.5), mul(sub(1.0, mul(th, th)), du))
    return add_(left, right)


_ACTIVATIONS = {"relu": _lib.RELU, "leaky_relu": _lib.LEAKY_RELU, "sigmoid": _lib.SIGMOID, "gelu": _lib.GELU}


def activation_backward(activation: str, x: HIPTensor, dout: HIPTensor, p: float = 0.0,
                        in_place: bool = False) -> HIPTensor:
    """dout f'(x) for 'relu', 'leaky_relu' (slope p), 'sigmoid', 'gelu' from the saved input x in one
    kernel (HIP-Activation-Node-backward).  With ``in_place`` the result overwrites dout."""
    d = dout if in_place else copy(dout)
    return nodes.forward("HIP-Activation-Node-backward", d, x, _ACTIVATIONS[activation], float(p))


def linear_backward(x: HIPTensor, w: HIPTensor, b: HIPTensor, dout: HIPTensor, activation: str | None = None,
                    fused: bool = True):
    """(dx, dw, db) of ``act(x . w + b)`` (HIP-Linear-Node, and HIP-Linear-Residual-Node whose
    residual passes ``dout`` through unchanged): dX = dZ W^T, dW = X^T dZ, dB = column sums of
    dZ, with dZ = dOUT for a plain layer and dOUT gelu'(Z), Z = X W + B recomputed (one product
    with the bias in its epilogue), for a GELU layer (``linear-gradients`` of the Lisp glue;
    MatMulNode's backward, ``base-impl/matrix-ops.lisp:10-15``).  ``fused=False`` composes
    gelu' node for node."""
    k, n = x.shape[-1], w.shape[-1]
    x2, d2 = reshape(x, -1, k), reshape(dout, -1, n)
    if activation == "gelu":
        if fused:
            z = linear(x2, w, b)
            dz = activation_backward("gelu", z, d2)
        else:
            z = add_(matmul(x2, w), b)
            dz = mul_(gelu_derivative(z), d2)
    elif activation is None:
        dz = d2
    else:
        raise ValueError("linear_backward: activation must be None or 'gelu'")
    dx = matmul(dz, t(w))
    dw = matmul(t(x2), dz)
    db = reshape(sum(dz, axis=0), n)
    return HIPTensor(list(x.shape), vec=dx.vec), dw, db


def softmax_backward_composed(y: HIPTensor, dout: HIPTensor, scale: float = 1.0) -> HIPTensor:
    """dx = scale y (dy - sum_j dy y) over the last axis node for node."""
    dot = sum(mul(dout, y), axis=-1, keepdims=True)
    dx = mul_(sub(dout, dot), y)
    return dx if scale == 1.0 else mul_(dx, float(scale))


def softmax_backward(y: HIPTensor, dout: HIPTensor, scale: float = 1.0, causal: bool = False,
                     in_place: bool = False) -> HIPTensor:
    """dx = scale y (dy - sum_j dy y) over the last axis from the saved output y in one kernel
    (HIP-Softmax-Node-backward; HIP-Causal-Softmax-Node-backward with ``causal``, which neither
    reads dout above the diagonal nor leaves dx unwritten there).  With ``in_place`` the result
    overwrites dout."""
    y, dout = to_contiguous(y), to_contiguous(dout)
    dx = dout if in_place else HIPTensor(list(y.shape), initial_element=None)
    if causal:
        return nodes.forward("HIP-Causal-Softmax-Node-backward", y, dout, dx, float(scale))
    nodes.forward("HIP-Softmax-Node-backward", y, dout, dx)
    return dx if scale == 1.0 else mul_(dx, float(scale))


def attention_backward(q: HIPTensor, k: HIPTensor, v: HIPTensor, dout: HIPTensor, scale: float | None = None,
                       causal: bool = False, dq: HIPTensor | None = None, dk: HIPTensor | None = None,
                       dv: HIPTensor | None = None, fused: bool = True, out: HIPTensor | None = None,
                       lse: HIPTensor | None = None):
    """(dq, dk, dv) of HIP-Attention-Node with the probabilities recomputed, as its :backward
    composes them: P = softmax(scale Q K^T [+ mask]), dV = P^T dO, dP = dO V^T,
    dS = scale P (dP - sum_j dP P), dQ = dS K, dK = dS^T Q.  Operands are
    (batch, heads, seq, head_dim) views whose last axis is contiguous; the optional outputs may be
    such views too (windows of one fused-projection gradient).  With a mask the two score-shaped
    products form their lower triangles only and dS K skips the tiles above the diagonal.
    ``fused=False`` takes the softmax gradient node for node and every product in full.
    With the forward pass's output ``out`` and row statistics ``lse`` (`attention(..., lse=)`) the
    whole backward is HIP-Attention-Node-backward instead: two launches, no (seq, seq) tensor."""
    hd = q.shape[-1]
    scale = 1.0 / math.sqrt(hd) if scale is None else float(scale)
    if out is not None and lse is not None:
        dq, dk, dv = (HIPTensor(list(t.shape), initial_element=None) if g is None else g
                      for t, g in ((q, dq), (k, dk), (v, dv)))
        same = lambda a, b: a.geometry()[1] == b.geometry()[1]  # noqa: E731
        if same(dout, out) and same(dq, q) and same(dk, k) and same(dv, v):
            return nodes.forward("HIP-Attention-Node-backward", q, k, v, out, dout, lse, dq, dk, dv, scale, causal)
        # operands laid out differently from the tensors they belong to: contiguous copies
        qc, kc, vc, oc, dc = (to_contiguous(t) for t in (q, k, v, out, dout))
        gq, gk, gv = (HIPTensor(list(q.shape), initial_element=None) for _ in range(3))
        nodes.forward("HIP-Attention-Node-backward", qc, kc, vc, oc, dc, lse, gq, gk, gv, scale, causal)
        return move_(dq, gq), move_(dk, gk), move_(dv, gv)
    tri = 1 if (causal and fused) else 0
    s = matmul(q, t(k), causal=tri)
    if causal:
        p = causal_softmax_fused(s, scale, out=s if fused else None)
    else:
        p = reshape(softmax_fused(reshape(mul_(s, scale), -1, s.shape[-1])), *s.shape)
    dv = matmul(t(p), dout, out=dv)
    dp = matmul(dout, t(v), causal=tri)
    if fused:
        ds = softmax_backward(p, dp, scale=scale, causal=causal, in_place=True)
    else:
        ds = softmax_backward_composed(p, dp, scale)
    dq = matmul(ds, k, out=dq, causal=2 if tri else 0)
    dk = matmul(t(ds), q, out=dk)
    return dq, dk, dv
