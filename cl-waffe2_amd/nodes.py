"""Node dispatch and the HIPTensor implementations (the ``define-impl`` layer).

Mirror of how a cl-waffe2 backend plugs in (``source/vm/nodes/defnode.lisp``):

* ``define_impl(node, device, reject_p)`` registers an implementation in
  ``DEVICE_FEATURES[device][node]`` (``defnode.lisp:428-571``, ``:535-538``);
* ``forward(node, *tensors)`` walks the priority list ``USING_BACKEND`` and
  takes the first device that has an implementation whose ``reject_p`` does not
  reject the dtype (``determine-facet-of-nodes``, ``defnode.lisp:215-232``);
  nothing matching raises ``NodeNotFound`` -- there is no silent fallback;
* each implementation returns its output tensor, as the VM requires
  (``source/vm/vm.lisp:144-150``).

The implementations below are what ``(define-impl (AddNode :device HIPTensor)
...)`` etc. do on the Lisp side: turn the tensors' views into one
``wf2hip_view2`` and make ONE library call per node, where the CPU backend emits
host loops around 1-D kernels (``source/backends/cpu/arithmetic.lisp:32-144``,
``mathematics.lisp:8-76``, ``matrix-ops.lisp:12-237``).
"""
from __future__ import annotations

import ctypes as C
import itertools
from contextlib import contextmanager

from . import lib as _lib
from .tensor import HIPTensor

NODE_NAMES = (
    "AddNode", "SubNode", "MulNode", "DivNode", "MoveTensorNode",
    "SinNode", "CosNode", "TanhNode", "LogENode", "ExpNode", "SqrtNode", "AbsNode",
    "TanNode", "ASinNode", "ACosNode", "ATanNode", "SinHNode", "CosHNode", "Log2Node", "Log10Node", "Log1pNode",
    "SignNode", "SquareNode", "ASinHNode", "ACosHNode", "ATanHNode",
    "ExptNode", "MatMulNode",
    "Where-Operation-Node", "Compare-Operation-Node",
    "MaxValue-Node", "MinValue-Node", "ArgMax-Node", "ArgMin-Node",
    "Im2ColNode", "Col2ImNode",
    # the define-op nodes of lisp/fusion.lisp (one kernel each)
    "HIP-Sum-Node", "HIP-Activation-Node", "HIP-Softmax-Node", "HIP-LayerNorm-Node", "HIP-Linear-Node",
    "HIP-Linear-Residual-Node", "HIP-Causal-Softmax-Node", "HIP-Attention-Node", "HIP-Softmax-Cross-Entropy-Node",
    "HIP-Unfold-Node",
    # the -backward nodes define-op generates for them, where the backward is one kernel too
    "HIP-Activation-Node-backward", "HIP-Softmax-Node-backward", "HIP-Causal-Softmax-Node-backward",
    "HIP-LayerNorm-Node-backward", "HIP-Attention-Node-backward", "HIP-Softmax-Cross-Entropy-Node-backward",
    # the node of the reference's GPT-2 example (examples/gpt-2/utils.lisp:68-72)
    "GPT2PositionalEmbedding",
)

DEVICE_FEATURES: dict[type, dict[str, tuple]] = {}
USING_BACKEND: list[type] = [HIPTensor]


class NodeNotFound(LookupError):
    """No device in the backend list implements the node (``node-not-found``)."""


def define_impl(node: str, device: type, reject_p=None):
    if node not in NODE_NAMES:
        raise ValueError(f"unknown AbstractNode {node}")

    def register(fn):
        DEVICE_FEATURES.setdefault(device, {})[node] = (fn, reject_p)
        return fn

    return register


@contextmanager
def with_devices(*devices):
    """``(with-devices (D1 D2 ...) ...)`` (``source/utils.lisp:7-17``)."""
    global USING_BACKEND
    saved = USING_BACKEND
    USING_BACKEND = list(devices)
    try:
        yield
    finally:
        USING_BACKEND = saved


def find_impl(node: str, dtype: str = "float"):
    for device in USING_BACKEND:
        entry = DEVICE_FEATURES.get(device, {}).get(node)
        if entry is None:
            continue
        fn, reject_p = entry
        if reject_p is not None and reject_p(dtype):
            continue
        return fn
    raise NodeNotFound(f"{node}: no implementation for dtype {dtype} among "
                       f"{[d.__name__ for d in USING_BACKEND]}")


def forward(node: str, *args, **kwargs):
    dtype = getattr(args[0], "dtype", "float")
    return find_impl(node, dtype)(*args, **kwargs)


# ---------------------------------------------------------------------------
# HIPTensor implementations
# ---------------------------------------------------------------------------

def _only_float(dtype) -> bool:
    """reject-p: only ``:float`` runs on the device (``supported-dtypes-are``,
    ``source/vm/nodes/utils.lisp:71-93``)."""
    return dtype != "float"


def view2(a: HIPTensor, b: HIPTensor) -> _lib.View2:
    sa, sta, oa = a._geom()
    sb, stb, ob = b._geom()
    if sa != sb:
        raise ValueError(f"shape mismatch: {list(sa)} and {list(sb)} (the node's :where is A[~] B[~] -> A[~])")
    v = _lib.View2()
    v.rank = len(sa)
    for r, (n, x, y) in enumerate(zip(sa, sta, stb)):
        v.shape[r] = n
        v.stride_a[r] = x
        v.stride_b[r] = y
    v.off_a = oa
    v.off_b = ob
    return v


def _binary(op):
    def impl(x: HIPTensor, y: HIPTensor) -> HIPTensor:
        v = view2(x, y)
        _lib.check(_lib.get().wf2hip_binary_nd(op, C.byref(v), C.c_void_p(x.ptr), C.c_void_p(y.ptr)))
        return x

    return impl


def _float_or_double(dtype) -> bool:
    """reject-p of the math and index nodes: the SIMD extension and BLAS cover
    :float and :double (``backends/cpu/mathematics.lisp:8-76``,
    ``matrix-ops.lisp:254-266``)."""
    return dtype not in ("float", "double")


def _run_unary(op, x: HIPTensor, out: HIPTensor, p: float) -> HIPTensor:
    if x.dtype != out.dtype:
        raise ValueError(f"dtype mismatch: {x.dtype} and {out.dtype}")
    v = view2(x, out)
    if x.dtype == "float":
        _lib.check(_lib.get().wf2hip_unary_nd(op, C.byref(v), C.c_void_p(x.ptr), C.c_void_p(out.ptr), p))
    else:
        _lib.check(_lib.get().wf2hip_unary_nd_typed(_lib.DTYPE_CODES[x.dtype], op, C.byref(v), C.c_void_p(x.ptr),
                                                    C.c_void_p(out.ptr), p))
    return out


def _unary(op):
    def impl(x: HIPTensor, out: HIPTensor) -> HIPTensor:
        return _run_unary(op, x, out, 0.0)

    return impl


def _binary_any_dtype(op):
    """The arithmetic and move nodes take every dtype (``backends/cpu/
    arithmetic.lisp:65-144`` dispatches on dtype inside the impl): :float goes to
    the kernels of the hot path, the rest to the typed entry point."""
    float_impl = _binary(op)

    def impl(x: HIPTensor, y: HIPTensor) -> HIPTensor:
        if x.dtype != y.dtype:
            raise ValueError(f"dtype mismatch: {x.dtype} and {y.dtype}")
        if x.dtype == "float":
            return float_impl(x, y)
        v = view2(x, y)
        _lib.check(_lib.get().wf2hip_binary_nd_typed(_lib.DTYPE_CODES[x.dtype], op, C.byref(v),
                                                    C.c_void_p(x.ptr), C.c_void_p(y.ptr)))
        return x

    return impl


for _name, _op in (("AddNode", _lib.ADD), ("SubNode", _lib.SUB), ("MulNode", _lib.MUL),
                   ("DivNode", _lib.DIV), ("MoveTensorNode", _lib.MOVE)):
    define_impl(_name, HIPTensor)(_binary_any_dtype(_op))

for _name, _op in (("SinNode", _lib.SIN), ("CosNode", _lib.COS), ("TanhNode", _lib.TANH),
                   ("LogENode", _lib.LOG), ("ExpNode", _lib.EXP), ("SqrtNode", _lib.SQRT),
                   ("AbsNode", _lib.ABS), ("TanNode", _lib.TAN), ("ASinNode", _lib.ASIN), ("ACosNode", _lib.ACOS),
                   ("ATanNode", _lib.ATAN), ("SinHNode", _lib.SINH), ("CosHNode", _lib.COSH),
                   ("Log2Node", _lib.LOG2), ("Log10Node", _lib.LOG10), ("Log1pNode", _lib.LOG1P),
                   # nodes the CPU backend leaves to LispTensor (base-impl/mathematics.lisp:131,147,217-219):
                   # with HIPTensor first in the backend list they must stay on the device
                   ("SignNode", _lib.SIGN), ("SquareNode", _lib.SQUARE), ("ASinHNode", _lib.ASINH),
                   ("ACosHNode", _lib.ACOSH), ("ATanHNode", _lib.ATANH)):
    define_impl(_name, HIPTensor, _float_or_double)(_unary(_op))


@define_impl("ExptNode", HIPTensor, _float_or_double)
def _expt(x: HIPTensor, out: HIPTensor, n: float) -> HIPTensor:
    return _run_unary(_lib.POW, x, out, float(n))


_CONDITIONS = {"=": _lib.EQ, "==": _lib.EQ, "<": _lib.LT, "<=": _lib.LE, ">": _lib.GT, ">=": _lib.GE}


def _condition(op) -> int:
    """The five predicates the SIMD extension implements
    (``backends/cpu/logical.lisp:26-33``); anything else has no device kernel."""
    if op in _CONDITIONS:
        return _CONDITIONS[op]
    raise NodeNotFound(f"no HIPTensor kernel for condition {op!r} (supported: = < <= > >=)")


@define_impl("Where-Operation-Node", HIPTensor)
def _where(x: HIPTensor, out: HIPTensor, condition, scal: float, true_then: float = 1.0,
           false_then: float = 0.0) -> HIPTensor:
    """``out <- (x condition scal) ? true-then : false-then``
    (``backends/cpu/logical.lisp:37-60``); x and out share one dtype."""
    if x.dtype != out.dtype:
        raise ValueError(f"dtype mismatch: {x.dtype} and {out.dtype}")
    v = view2(x, out)
    if x.dtype == "float":
        _lib.check(_lib.get().wf2hip_where_nd(_condition(condition), C.byref(v), C.c_void_p(x.ptr),
                                              C.c_void_p(out.ptr), float(scal), float(true_then),
                                              float(false_then)))
    else:
        _lib.check(_lib.get().wf2hip_where_nd_typed(_lib.DTYPE_CODES[x.dtype], _condition(condition), C.byref(v),
                                                    C.c_void_p(x.ptr), C.c_void_p(out.ptr), float(scal),
                                                    float(true_then), float(false_then)))
    return out


def view3(a: HIPTensor, b: HIPTensor, c: HIPTensor) -> _lib.View3:
    sa, sta, oa = a.geometry()
    sb, stb, ob = b.geometry()
    sc, stc, oc = c.geometry()
    if not (sa == sb == sc):
        raise ValueError(f"shape mismatch: {sa}, {sb} and {sc}")
    v = _lib.View3()
    v.rank = len(sa)
    for r, (n, x, y, z) in enumerate(zip(sa, sta, stb, stc)):
        v.shape[r] = n
        v.stride_a[r] = x
        v.stride_b[r] = y
        v.stride_c[r] = z
    v.off_a, v.off_b, v.off_c = oa, ob, oc
    return v


@define_impl("Compare-Operation-Node", HIPTensor)
def _compare(x: HIPTensor, y: HIPTensor, out: HIPTensor, condition, true_then: float = 1.0,
             false_then: float = 0.0) -> HIPTensor:
    """``out <- (x condition y) ? true-then : false-then``
    (``backends/cpu/logical.lisp:62-84``); all three share one dtype."""
    if not (x.dtype == y.dtype == out.dtype):
        raise ValueError(f"dtype mismatch: {x.dtype}, {y.dtype} and {out.dtype}")
    v = view3(x, y, out)
    if x.dtype == "float":
        _lib.check(_lib.get().wf2hip_compare_nd(_condition(condition), C.byref(v), C.c_void_p(x.ptr),
                                                C.c_void_p(y.ptr), C.c_void_p(out.ptr),
                                                float(true_then), float(false_then)))
    else:
        _lib.check(_lib.get().wf2hip_compare_nd_typed(_lib.DTYPE_CODES[x.dtype], _condition(condition), C.byref(v),
                                                      C.c_void_p(x.ptr), C.c_void_p(y.ptr), C.c_void_p(out.ptr),
                                                      float(true_then), float(false_then)))
    return out


def _select(op, index: bool):
    def impl(x: HIPTensor, out: HIPTensor) -> HIPTensor:
        """``A[~] OUT[out-size] -> OUT``: one element of OUT per trailing run of A
        (``base-impl/matrix-ops.lisp:200-383``; CPU forwards
        ``backends/cpu/matrix-ops.lisp:240-369``)."""
        xs, xst, xo = x.geometry()
        os_, ost, oo = out.geometry()
        if len(xs) != len(os_) or xs[:-1] != os_[:-1] or os_[-1] != 1:
            raise ValueError(f"{x.shape} selects into {xs[:-1] + [1]}, not {out.shape}")
        if out.dtype != ("uint32" if index else x.dtype):
            raise ValueError("ArgMax/ArgMin write :uint32, MaxValue/MinValue the dtype of A")
        v = _lib.View2()
        v.rank = max(len(xs) - 1, 1)
        v.shape[0], v.stride_a[0], v.stride_b[0] = 1, 0, 0
        for r in range(len(xs) - 1):
            v.shape[r], v.stride_a[r], v.stride_b[r] = xs[r], xst[r], ost[r]
        v.off_a, v.off_b = xo, oo
        if x.dtype == "float":
            _lib.check(_lib.get().wf2hip_select_nd(op, C.byref(v), xs[-1], xst[-1], C.c_void_p(x.ptr),
                                                   C.c_void_p(out.ptr)))
        else:
            _lib.check(_lib.get().wf2hip_select_nd_typed(_lib.DTYPE_CODES[x.dtype], op, C.byref(v), xs[-1], xst[-1],
                                                         C.c_void_p(x.ptr), C.c_void_p(out.ptr)))
        return out

    return impl


# the value nodes take every dtype (waffe2_<prefix>{max,min}, backends/cpu/matrix-ops.lisp:323-369)
define_impl("MaxValue-Node", HIPTensor)(_select(_lib.MAXVALUE, False))
define_impl("MinValue-Node", HIPTensor)(_select(_lib.MINVALUE, False))
define_impl("ArgMax-Node", HIPTensor, _float_or_double)(_select(_lib.ARGMAX, True))
define_impl("ArgMin-Node", HIPTensor, _float_or_double)(_select(_lib.ARGMIN, True))


def _unfold_args(x_shape, col_shape, stride, padding, dilation):
    N, Cc, H, W = x_shape
    n2, c2, kh, kw, ho, wo = col_shape
    if (N, Cc) != (n2, c2):
        raise ValueError(f"X {x_shape} and Col {col_shape} disagree on N, C")
    return [N, Cc, H, W, ho, wo, kh, kw, padding[0], padding[1], stride[0], stride[1], dilation[0], dilation[1]]


@define_impl("HIP-Sum-Node", HIPTensor, _only_float)
def _sum_node(out: HIPTensor, x: HIPTensor, divisor: float = 1.0) -> HIPTensor:
    """``Out[~] X[~] -> Out[~]`` with `out` viewed ``(:broadcast n)`` on the reduced axes:
    out <- sum of x over those axes / divisor, overwriting `out`.  One node for the
    MulNode-by-0, AddNode and DivNode of ``!sum`` / ``!mean``
    (``base-impl/reduction.lisp:5-136``); its backward is theirs (the gradient
    broadcast over the reduced axes, divided by `divisor`)."""
    v = view2(out, x)
    _lib.check(_lib.get().wf2hip_sum_nd(C.byref(v), C.c_void_p(out.ptr), C.c_void_p(x.ptr), float(divisor)))
    return out


@define_impl("Im2ColNode", HIPTensor, _only_float)
def _im2col(x: HIPTensor, col: HIPTensor, stride, padding, dilation) -> HIPTensor:
    """``X[N C H W] Col[N C k-h k-w h-out w-out] -> Col`` with X already padded
    (``base-impl/unfold.lisp``; CPU forward ``backends/cpu/im2col.lisp:3-26``)."""
    if not (x.is_contiguous() and col.is_contiguous()):
        raise ValueError("Im2ColNode takes contiguous tensors (the CPU kernel indexes the storage directly)")
    args = _unfold_args(x.shape, col.shape, stride, padding, dilation)
    _lib.check(_lib.get().wf2hip_im2col_f32(C.c_void_p(col.ptr), *args, C.c_void_p(x.ptr)))
    return col


@define_impl("Col2ImNode", HIPTensor, _only_float)
def _col2im(col: HIPTensor, x: HIPTensor, stride, padding, dilation) -> HIPTensor:
    """``Col[N C k-h k-w h-out w-out] X[N C H W] -> X``: X is overwritten with the
    sum of the columns (``backends/cpu/im2col.lisp:28-50``)."""
    if not (x.is_contiguous() and col.is_contiguous()):
        raise ValueError("Col2ImNode takes contiguous tensors")
    args = _unfold_args(x.shape, col.shape, stride, padding, dilation)
    _lib.check(_lib.get().wf2hip_col2im_f32(C.c_void_p(col.ptr), *args, C.c_void_p(x.ptr)))
    return x


@define_impl("HIP-Unfold-Node", HIPTensor, _only_float)
def _unfold_node(x: HIPTensor, out: HIPTensor, kernel_size, stride, padding) -> HIPTensor:
    """``X[N C H W] OUT[(N h-out w-out) (C k-h k-w)] -> OUT``: ``unfold`` with dilation 1
    (``source/nn/im2col.lisp:51-95``: padding, Im2ColNode, permutation, reshape) as one kernel."""
    if len(x.shape) != 4:
        raise ValueError("HIP-Unfold-Node takes a [N C H W] tensor")
    _require_rows("HIP-Unfold-Node: x", x)
    N, Cc, H, W = x.shape
    (kh, kw), (sh, sw), (ph, pw) = ((int(v[0]), int(v[1])) for v in (kernel_size, stride, padding))
    if min(kh, kw, sh, sw) < 1 or min(ph, pw) < 0 or H + 2 * ph < kh or W + 2 * pw < kw:
        raise ValueError(f"HIP-Unfold-Node: kernel {kh, kw}, stride {sh, sw}, padding {ph, pw} on a {H} x {W} image")
    h_out, w_out = (H + 2 * ph - kh) // sh + 1, (W + 2 * pw - kw) // sw + 1
    _require_rows("HIP-Unfold-Node: out", out, [N * h_out * w_out, Cc * kh * kw])
    _lib.check(_lib.get().wf2hip_unfold_f32(N, Cc, H, W, kh, kw, sh, sw, ph, pw, C.c_void_p(x.ptr), C.c_void_p(out.ptr)))
    return out


def _matrix_geometry(t: HIPTensor, what: str):
    """Batch shape/strides, start offset and the leading dimension of the last
    two axes.  The last axis must be unit-stride (the CPU backend reads ldX as
    the last-axis size of the untransposed tensor, matrix-ops.lisp:40-47)."""
    shape, strides, off = t.geometry()
    if len(shape) < 2:
        raise ValueError(f"MatMulNode: {what} needs rank >= 2")
    if shape[-1] > 1 and strides[-1] != 1:
        raise ValueError(f"MatMulNode: {what} must be contiguous along its last axis; "
                         "materialise it with to_contiguous first")
    ld = strides[-2] if shape[-2] > 1 else max(shape[-1], 1)
    if ld < shape[-1]:
        raise ValueError(f"MatMulNode: {what} rows overlap (broadcast rows are not supported)")
    return shape, strides, off, ld


@define_impl("MatMulNode", HIPTensor, _float_or_double)
def _matmul(a: HIPTensor, b: HIPTensor, out: HIPTensor, trans_a: bool = False,
            trans_b: bool = False, bias: HIPTensor | None = None,
            residual: HIPTensor | None = None, activation: str | None = None,
            causal: int = 0) -> HIPTensor:
    """``C[~ i k] = A[~ i j] . B[~ j k]`` through the operand-swapped
    column-major call of ``expand-gemm-form-column``
    (``backends/cpu/matrix-ops.lisp:12-112``): sgemm(transB, transA, n, m, k, 1,
    B, ldb, A, lda, 0, C, ldc).  ``a``/``b`` are the tensors as stored (i.e.
    untransposed); batch axes may be broadcast (stride 0) on either operand.

    ``bias`` / ``activation`` / ``residual`` / ``causal`` select the fused
    epilogue of ``wf2hip_matmul_fused`` (not part of MatMulNode: what a
    ``define-bypass`` fusion of MatMulNode + AddNode (+ !gelu) would call).

    :double operands take ``wf2hip_dgemm_strided_batched_2d`` (the CPU backend's
    dgemm_ branch of the same expansion); the fused epilogues are :float only."""
    if not (a.dtype == b.dtype == out.dtype):
        raise ValueError(f"MatMulNode: dtype mismatch: {a.dtype}, {b.dtype} -> {out.dtype}")
    sa, sta, oa, lda = _matrix_geometry(a, "A")
    sb, stb, ob, ldb = _matrix_geometry(b, "B")
    sc, stc, oc, ldc = _matrix_geometry(out, "C")
    m, n = sc[-2], sc[-1]
    k = sa[-2] if trans_a else sa[-1]
    if (sa[-1] if trans_a else sa[-2]) != m or (sb[-1] if trans_b else sb[-2]) != k or \
            (sb[-2] if trans_b else sb[-1]) != n:
        raise ValueError(f"MatMulNode: shapes {sa} {'T' if trans_a else ''} x {sb} "
                         f"{'T' if trans_b else ''} -> {sc} do not agree")
    batch_shape = sc[:-2]
    if sa[:-2] != batch_shape or sb[:-2] != batch_shape:
        raise ValueError("MatMulNode: batch axes differ; view the smaller operand with (:broadcast n)")
    fused = bias is not None or residual is not None or activation is not None or causal
    if fused and a.dtype != "float":
        raise ValueError("MatMulNode: bias / activation / residual / causal epilogues are :float only")
    tensors = [sta, stb, stc]
    ores = ldres = 0
    if residual is not None:
        sr, strd, ores, ldres = _matrix_geometry(residual, "residual")
        if sr != sc:
            raise ValueError(f"residual shape {sr} differs from the product's {sc}")
        tensors.append(strd)
    if bias is not None and (bias.shape != [n] or not bias.is_contiguous()):
        raise ValueError(f"bias must be a contiguous vector of {n} elements")
    if activation not in (None, "gelu"):
        raise ValueError("activation must be None or 'gelu'")
    lib = _lib.get()
    ta = b"C" if trans_a else b"N"
    tb = b"C" if trans_b else b"N"

    def launch(offs, inner, outer):
        (count, s3), (count2, s3o) = inner, outer
        if not fused:
            gemm = lib.wf2hip_sgemm_strided_batched_2d if a.dtype == "float" \
                else lib.wf2hip_dgemm_strided_batched_2d
            w = a.itemsize
            _lib.check(gemm(
                tb, ta, n, m, k, 1.0,
                C.c_void_p(b.ptr + w * offs[1]), ldb, s3[1], s3o[1],
                C.c_void_p(a.ptr + w * offs[0]), lda, s3[0], s3o[0],
                0.0, C.c_void_p(out.ptr + w * offs[2]), ldc, s3[2], s3o[2], count, count2))
            return
        d = _lib.MatmulDesc()
        d.trans_a, d.trans_b = int(trans_a), int(trans_b)
        d.activation = 1 if activation == "gelu" else 0
        d.causal = int(causal)
        d.m, d.n, d.k = m, n, k
        d.lda, d.ldb, d.ldc = lda, ldb, ldc
        d.batch, d.batch2 = count, count2
        d.stride_a, d.stride_a2 = s3[0], s3o[0]
        d.stride_b, d.stride_b2 = s3[1], s3o[1]
        d.stride_c, d.stride_c2 = s3[2], s3o[2]
        d.bias = bias.ptr if bias is not None else None
        if residual is not None:
            d.residual = residual.ptr + 4 * offs[3]
            d.ld_residual, d.stride_residual, d.stride_residual2 = ldres, s3[3], s3o[3]
        d.alpha = 1.0
        _lib.check(lib.wf2hip_matmul_fused(C.byref(d), C.c_void_p(a.ptr + 4 * offs[0]),
                                           C.c_void_p(b.ptr + 4 * offs[1]),
                                           C.c_void_p(out.ptr + 4 * offs[2])))

    # Fold the batch axes, innermost first, into at most two strided axes per
    # launch (the library takes two batch levels); anything beyond that is
    # walked on the host like the CPU backend walks every batch index.
    # Extent-1 axes carry no information.
    keep = [i for i, n_ in enumerate(batch_shape) if n_ != 1]
    batch_shape = [batch_shape[i] for i in keep]
    tensors = [[st[i] for i in keep] for st in tensors]
    start = [oa, ob, oc] + ([ores] if residual is not None else [])

    def fold(last):
        """Merge axes last, last-1, ... while they form one strided run for
        every tensor (0 == 0 x count holds for a broadcast operand)."""
        count = batch_shape[last]
        s3 = [st[last] for st in tensors]
        first = last
        while first > 0 and all(st[first - 1] == s * count for st, s in zip(tensors, s3)):
            first -= 1
            count *= batch_shape[first]
        return first, (count, s3)

    none = (1, [0] * len(tensors))
    if not batch_shape:
        launch(start, none, none)
        return out
    first, inner = fold(len(batch_shape) - 1)
    outer = none
    if first > 0:
        first, outer = fold(first - 1)
    if inner[0] * outer[0] > 65535:
        raise ValueError("MatMulNode: more than 65535 matrices in one launch")
    outer_shape = batch_shape[:first]

    # (an explicit product instead of a recursive closure: a function that
    # refers to itself is a reference cycle, which would keep the operands --
    # and their device memory -- alive until the cyclic collector runs)
    for index in itertools.product(*[range(n_) for n_ in outer_shape]):
        launch([o + sum(i * st[ax] for ax, i in enumerate(index)) for o, st in zip(start, tensors)],
               inner, outer)
    return out


# ---------------------------------------------------------------------------
# the define-op nodes of lisp/fusion.lisp: one kernel per node
# ---------------------------------------------------------------------------

def _require_rows(what: str, t: HIPTensor, shape=None) -> None:
    """The row kernels take base pointers and a row count: the tensor must be :float,
    contiguous and start at its storage (a view would be read or written elsewhere)."""
    if t.dtype != "float":
        raise ValueError(f"{what} must be :float, got :{t.dtype}")
    _, _, off = t.geometry()
    if not t.is_contiguous() or off != 0:
        raise ValueError(f"{what} must be a contiguous tensor that starts at its storage; "
                         "materialise the view with to_contiguous first")
    if shape is not None and list(t.shape) != list(shape):
        raise ValueError(f"{what} has shape {t.shape}, expected {list(shape)}")


@define_impl("HIP-Activation-Node", HIPTensor, _only_float)
def _activation_node(x: HIPTensor, out: HIPTensor, op: int, p: float = 0.0) -> HIPTensor:
    """``X[~] OUT[~] -> OUT[~]``: ReLU / leaky ReLU / sigmoid / GELU as one kernel."""
    return _run_unary(op, x, out, float(p))


@define_impl("HIP-Activation-Node-backward", HIPTensor, _only_float)
def _activation_backward_node(dout: HIPTensor, x: HIPTensor, op: int, p: float = 0.0) -> HIPTensor:
    """``DOUT[~] X[~] -> DOUT[~]``: dout <- dout f'(x) in place, x the saved input."""
    v = view2(dout, x)
    _lib.check(_lib.get().wf2hip_activation_backward_nd(op, C.byref(v), C.c_void_p(dout.ptr), C.c_void_p(x.ptr),
                                                       float(p)))
    return dout


def _softmax_backward(name: str, y: HIPTensor, dout: HIPTensor, dx: HIPTensor, scale: float, causal: bool) -> HIPTensor:
    _require_rows(f"{name}: y", y)
    _require_rows(f"{name}: dout", dout, y.shape)
    _require_rows(f"{name}: dx", dx, y.shape)
    cols = y.shape[-1]
    if causal and (len(y.shape) < 2 or y.shape[-2] != cols):
        raise ValueError(f"{name} takes square score matrices, got {y.shape}")
    rows = y.size // max(cols, 1)
    _lib.check(_lib.get().wf2hip_softmax_backward_rows_f32(rows, cols, C.c_void_p(y.ptr), cols, C.c_void_p(dout.ptr),
                                                          cols, C.c_void_p(dx.ptr), cols, float(scale),
                                                          cols if causal else 0))
    return dx


@define_impl("HIP-Softmax-Node-backward", HIPTensor, _only_float)
def _softmax_backward_node(y: HIPTensor, dout: HIPTensor, dx: HIPTensor) -> HIPTensor:
    """``Y[rows cols] DOUT[rows cols] DX[rows cols] -> DX``: y (dout - sum_j dout y); dx may be dout."""
    return _softmax_backward("HIP-Softmax-Node-backward", y, dout, dx, 1.0, False)


@define_impl("HIP-Causal-Softmax-Node-backward", HIPTensor, _only_float)
def _causal_softmax_backward_node(y: HIPTensor, dout: HIPTensor, dx: HIPTensor, scale: float = 1.0) -> HIPTensor:
    """``Y[matrices seq seq] DOUT[...] DX[...] -> DX``: scale y (dout - sum_j dout y) on and below the
    diagonal (dout is not read above it), 0 above."""
    return _softmax_backward("HIP-Causal-Softmax-Node-backward", y, dout, dx, scale, True)


@define_impl("HIP-LayerNorm-Node-backward", HIPTensor, _only_float)
def _layernorm_backward_node(x: HIPTensor, g: HIPTensor, dout: HIPTensor, dx: HIPTensor, dg: HIPTensor,
                             db: HIPTensor, eps: float = 1.0e-5) -> HIPTensor:
    """``X[rows cols] G[cols] DOUT[rows cols] DX[rows cols] DG[cols] DB[cols] -> DX DG DB``."""
    cols = x.shape[-1]
    name = "HIP-LayerNorm-Node-backward"
    _require_rows(f"{name}: x", x)
    _require_rows(f"{name}: dout", dout, x.shape)
    _require_rows(f"{name}: dx", dx, x.shape)
    for what, t in (("gamma", g), ("dgamma", dg), ("dbeta", db)):
        _require_rows(f"{name}: {what}", t, [cols])
    rows = x.size // max(cols, 1)
    _lib.check(_lib.get().wf2hip_layernorm_backward_f32(rows, cols, C.c_void_p(x.ptr), C.c_void_p(g.ptr),
                                                       C.c_void_p(dout.ptr), float(eps), C.c_void_p(dx.ptr),
                                                       C.c_void_p(dg.ptr), C.c_void_p(db.ptr)))
    return dx


@define_impl("HIP-Softmax-Node", HIPTensor, _only_float)
def _softmax_node(x: HIPTensor, out: HIPTensor) -> HIPTensor:
    """``X[rows cols] OUT[rows cols] -> OUT``: max-subtracted softmax over the last axis."""
    _require_rows("HIP-Softmax-Node: x", x)
    _require_rows("HIP-Softmax-Node: out", out, x.shape)
    cols = x.shape[-1]
    rows = x.size // max(cols, 1)
    _lib.check(_lib.get().wf2hip_softmax_rows_f32(rows, cols, C.c_void_p(x.ptr), cols, C.c_void_p(out.ptr), cols))
    return out


@define_impl("HIP-Softmax-Cross-Entropy-Node", HIPTensor, _only_float)
def _softmax_cross_entropy_node(x: HIPTensor, labels: HIPTensor, z: HIPTensor, out: HIPTensor,
                                delta: float = 1.0e-7) -> HIPTensor:
    """``X[rows cols] Labels[rows cols] Z[rows cols] OUT[rows cols] -> OUT``: Softmax-Cross-Entropy-Node
    (``source/nn/criterion.lisp:90-126``) as one kernel.  z <- softmax over the last axis (what the node
    saves for its backward), out <- -1 (labels log(z + delta))."""
    name = "HIP-Softmax-Cross-Entropy-Node"
    _require_rows(f"{name}: x", x)
    for what, t in (("labels", labels), ("z", z), ("out", out)):
        _require_rows(f"{name}: {what}", t, x.shape)
    cols = x.shape[-1]
    rows = x.size // max(cols, 1)
    _lib.check(_lib.get().wf2hip_softmax_cross_entropy_f32(rows, cols, C.c_void_p(x.ptr), C.c_void_p(labels.ptr),
                                                          float(delta), C.c_void_p(z.ptr), C.c_void_p(out.ptr)))
    return out


@define_impl("HIP-Softmax-Cross-Entropy-Node-backward", HIPTensor, _only_float)
def _softmax_cross_entropy_backward_node(dout: HIPTensor, z: HIPTensor, labels: HIPTensor, dx: HIPTensor) -> HIPTensor:
    """``DOUT[rows cols] Z[rows cols] Labels[rows cols] DX[rows cols] -> DX``: sce-diff-static
    (``source/nn/criterion.lisp:82-88``), (dout (z - labels)) / batch with batch the second-to-last extent
    of z.  A one-element ``dout`` is the number every element uses (the gradient under a !sum or !mean of
    the loss).  dx may be dout or z."""
    name = "HIP-Softmax-Cross-Entropy-Node-backward"
    _require_rows(f"{name}: z", z)
    _require_rows(f"{name}: labels", labels, z.shape)
    _require_rows(f"{name}: dx", dx, z.shape)
    scalar = dout.size == 1 and z.size != 1
    _require_rows(f"{name}: dout", dout, None if scalar else z.shape)
    batch = float(z.shape[-2]) if len(z.shape) >= 2 else 1.0
    _lib.check(_lib.get().wf2hip_softmax_cross_entropy_backward_f32(z.size, C.c_void_p(dout.ptr), int(scalar),
                                                                   C.c_void_p(z.ptr), C.c_void_p(labels.ptr), batch,
                                                                   C.c_void_p(dx.ptr)))
    return dx


@define_impl("HIP-LayerNorm-Node", HIPTensor, _only_float)
def _layernorm_node(x: HIPTensor, g: HIPTensor, b: HIPTensor, out: HIPTensor, eps: float = 1.0e-5) -> HIPTensor:
    """``X[rows cols] G[cols] B[cols] OUT[rows cols] -> OUT``."""
    cols = x.shape[-1]
    _require_rows("HIP-LayerNorm-Node: x", x)
    _require_rows("HIP-LayerNorm-Node: out", out, x.shape)
    _require_rows("HIP-LayerNorm-Node: gamma", g, [cols])
    _require_rows("HIP-LayerNorm-Node: beta", b, [cols])
    rows = x.size // max(cols, 1)
    _lib.check(_lib.get().wf2hip_layernorm_rows_f32(rows, cols, C.c_void_p(x.ptr), C.c_void_p(g.ptr),
                                                   C.c_void_p(b.ptr), float(eps), C.c_void_p(out.ptr)))
    return out


@define_impl("HIP-Linear-Node", HIPTensor, _only_float)
def _linear_node(x: HIPTensor, w: HIPTensor, b: HIPTensor, out: HIPTensor, activation: str | None = None) -> HIPTensor:
    """``X[rows k] W[k n] B[n] OUT[rows n] -> OUT``: act(x . w + b) as one product."""
    return _matmul(x, w, out, bias=b, activation=activation)


@define_impl("HIP-Linear-Residual-Node", HIPTensor, _only_float)
def _linear_residual_node(x: HIPTensor, w: HIPTensor, b: HIPTensor, r: HIPTensor, out: HIPTensor) -> HIPTensor:
    """``X[rows k] W[k n] B[n] R[rows n] OUT[rows n] -> OUT``: x . w + b + r as one product."""
    return _matmul(x, w, out, bias=b, residual=r)


@define_impl("HIP-Causal-Softmax-Node", HIPTensor, _only_float)
def _causal_softmax_node(x: HIPTensor, out: HIPTensor, scale: float = 1.0) -> HIPTensor:
    """``X[matrices seq seq] OUT[...] -> OUT``: softmax over j <= i of scale x[m, i, j], 0 above the diagonal."""
    _require_rows("HIP-Causal-Softmax-Node: x", x)
    _require_rows("HIP-Causal-Softmax-Node: out", out, x.shape)
    seq = x.shape[-1]
    if len(x.shape) < 2 or x.shape[-2] != seq:
        raise ValueError(f"HIP-Causal-Softmax-Node takes square score matrices, got {x.shape}")
    _lib.check(_lib.get().wf2hip_causal_softmax_f32(x.size // max(seq * seq, 1), seq, C.c_void_p(x.ptr),
                                                   C.c_void_p(out.ptr), float(scale)))
    return out


def _attention_desc(name: str, q, k, v, o, scale: float, causal: bool):
    """The descriptor of four (batch, heads, seq, head_dim) views and their start addresses."""
    if not (len(q.shape) == 4 and list(q.shape) == list(k.shape) == list(v.shape) == list(o.shape)):
        raise ValueError(f"{name} expects (batch, heads, seq, head_dim) tensors of one shape")
    B, H, T, hd = q.shape
    d = _lib.AttentionDesc()
    d.batch, d.heads, d.seq, d.head_dim = B, H, T, hd
    ptrs = []
    for t, field in ((q, d.q_stride), (k, d.k_stride), (v, d.v_stride), (o, d.o_stride)):
        _, strides, off = t.geometry()
        if hd > 1 and strides[3] != 1:
            raise ValueError(f"{name}: the head_dim axis must be contiguous")
        for a in range(3):
            field[a] = strides[a]
        ptrs.append(C.c_void_p(t.ptr + 4 * off))
    d.scale = float(scale)
    d.causal = 1 if causal else 0
    return d, ptrs


def _same_layout(name: str, what: str, t: HIPTensor, like: HIPTensor):
    """`t` must be addressed like `like` (the library reads one set of strides for both)."""
    if list(t.shape) != list(like.shape) or t.geometry()[1] != like.geometry()[1]:
        raise ValueError(f"{name}: {what} must have the shape and strides of the tensor it belongs to")
    return C.c_void_p(t.ptr + 4 * t.geometry()[2])


@define_impl("HIP-Attention-Node", HIPTensor, _only_float)
def _attention_node(q: HIPTensor, k: HIPTensor, v: HIPTensor, out: HIPTensor, scale: float,
                    causal: bool = False, lse: HIPTensor | None = None) -> HIPTensor:
    """``Q K V OUT[batch heads seq dim] -> OUT``: softmax(scale q k^T [+ mask]) v in one kernel.  `lse`, a
    contiguous (batch, heads, seq) tensor, receives the row statistics the backward node reads."""
    d, ptrs = _attention_desc("HIP-Attention-Node", q, k, v, out, scale, causal)
    if lse is None:
        _lib.check(_lib.get().wf2hip_attention_f32(C.byref(d), *ptrs))
    else:
        _require_rows("HIP-Attention-Node: lse", lse, list(q.shape[:3]))
        _lib.check(_lib.get().wf2hip_attention_forward_f32(C.byref(d), *ptrs, C.c_void_p(lse.ptr)))
    return out


@define_impl("HIP-Attention-Node-backward", HIPTensor, _only_float)
def _attention_backward_node(q: HIPTensor, k: HIPTensor, v: HIPTensor, out: HIPTensor, dout: HIPTensor,
                             lse: HIPTensor, dq: HIPTensor, dk: HIPTensor, dv: HIPTensor, scale: float,
                             causal: bool = False):
    """``Q K V OUT DOUT LSE DQ DK DV -> DQ DK DV``: the three gradients without a (seq, seq) tensor.  dout
    is addressed like out, dq / dk / dv like q / k / v."""
    name = "HIP-Attention-Node-backward"
    d, ptrs = _attention_desc(name, q, k, v, out, scale, causal)
    _require_rows(f"{name}: lse", lse, list(q.shape[:3]))
    extra = [_same_layout(name, "dout", dout, out), C.c_void_p(lse.ptr), _same_layout(name, "dq", dq, q),
             _same_layout(name, "dk", dk, k), _same_layout(name, "dv", dv, v)]
    _lib.check(_lib.get().wf2hip_attention_backward_f32(C.byref(d), *ptrs, *extra))
    return dq, dk, dv


@define_impl("GPT2PositionalEmbedding", HIPTensor, _only_float)
def _gpt2_positional_embedding(ctx: HIPTensor, wte: HIPTensor, wpe: HIPTensor, out: HIPTensor) -> HIPTensor:
    """``ctx[N sentence-length] wte[vocab-size embedding-size] wpe[n-ctx embedding-size]
    ctx-out[N sentence-length embedding-size] -> ctx-out``: out <- wte[round(ctx)] + wpe[position]
    (``examples/gpt-2/utils.lisp:68-110``; the example implements it for LispTensor only)."""
    name = "GPT2PositionalEmbedding"
    if len(ctx.shape) != 2 or len(wte.shape) != 2 or len(wpe.shape) != 2:
        raise ValueError(f"{name}: ctx, wte, wpe must be matrices")
    n, t = ctx.shape
    vocab, dim = wte.shape
    _require_rows(f"{name}: ctx", ctx)
    _require_rows(f"{name}: wte", wte)
    _require_rows(f"{name}: wpe", wpe, [wpe.shape[0], dim])
    _require_rows(f"{name}: ctx-out", out, [n, t, dim])
    _lib.check(_lib.get().wf2hip_embedding_add_f32(n * t, t, dim, C.c_void_p(ctx.ptr), C.c_void_p(wte.ptr), vocab,
                                                  C.c_void_p(wpe.ptr), wpe.shape[0], C.c_void_p(out.ptr)))
    return out
