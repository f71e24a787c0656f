"""Convolution and pooling as the reference composes them from unfold.

``source/nn/conv.lisp:90-104`` (apply-conv2d) and ``source/nn/pool.lisp:83-105``
(MaxPool2D / AvgPool2D): every step is one of the backend's nodes -- padding
(MoveTensorNode into a view), Im2ColNode, permute / reshape copies, MatMulNode,
AddNode, MaxValue-Node or the !mean composition -- so the layers run on the
device without a kernel of their own.
"""
from __future__ import annotations

from . import functional as F
from . import nodes
from .tensor import HIPTensor


def _pair(v):
    return (int(v), int(v)) if isinstance(v, int) else (int(v[0]), int(v[1]))


def conv2d(x: HIPTensor, weight: HIPTensor, bias: HIPTensor | None = None, stride=1, padding=0,
           dilation=1) -> HIPTensor:
    """``(call (Conv2D c-in c-out kernel-size ...) x)``: ``x`` is ``[N C_in H W]``,
    ``weight`` ``[C_out C_in k-h k-w]``, the result ``[N C_out H_out W_out]`` (a
    permuted view of the ``[N H_out W_out C_out]`` product, as in the reference)."""
    stride, padding, dilation = _pair(stride), _pair(padding), _pair(dilation)
    N, _, H, W = x.shape
    c_out, _, kh, kw = weight.shape
    h_out = F.conv_out_size(H, padding[0], dilation[0], kh, stride[0])
    w_out = F.conv_out_size(W, padding[1], dilation[1], kw, stride[1])
    col = F.unfold(x, dilation, (kh, kw), stride, padding)          # [(N h w) (C k-h k-w)]
    col_w = F.reshape(weight, c_out, -1)
    out = F.matmul(col, F.t(col_w))                                  # [(N h w) C_out]
    if bias is not None:
        out = F.add(out, bias)
    return F.reshape(out, N, h_out, w_out, c_out).permute(0, 3, 1, 2)


def _pool(x: HIPTensor, kernel_size, stride, padding, reduce) -> HIPTensor:
    kernel_size, stride, padding = _pair(kernel_size), _pair(stride), _pair(padding)
    N, Cc, H, W = x.shape
    h_out = (H + 2 * padding[0] - kernel_size[0]) // stride[0] + 1   # pool-out-size, pool.lisp:19-21
    w_out = (W + 2 * padding[1] - kernel_size[1]) // stride[1] + 1
    col = F.unfold(x, (1, 1), kernel_size, stride, padding)
    windows = F.reshape(col, -1, kernel_size[0] * kernel_size[1])   # [(N h w C) (k-h k-w)]
    red = reduce(windows)
    return F.reshape(red, N, h_out, w_out, Cc).permute(0, 3, 1, 2)


def max_pool2d(x: HIPTensor, kernel_size, stride=None, padding=0) -> HIPTensor:
    """``MaxPool2D`` (pool.lisp:83-93); padded positions hold 0, as in the
    reference."""
    return _pool(x, kernel_size, kernel_size if stride is None else stride, padding,
                 lambda w: F.max(w, axis=1))


def avg_pool2d(x: HIPTensor, kernel_size, stride=None, padding=0) -> HIPTensor:
    """``AvgPool2D`` (pool.lisp:95-105)."""
    return _pool(x, kernel_size, kernel_size if stride is None else stride, padding,
                 lambda w: F.mean(w, axis=1))


# ---------------------------------------------------------------------------
# backward of the layers above, as the nodes' own backward definitions compose it
# ---------------------------------------------------------------------------

def conv2d_backward(x: HIPTensor, weight: HIPTensor, dout: HIPTensor, stride=1, padding=0, bias: bool = True):
    """``(dx, dweight, dbias)`` of :func:`conv2d` for the upstream gradient ``dout[N C_out H_out W_out]``:
    the permutation of the output undone, MatMulNode's two backward products (dY^T . col and dY . W,
    ``base-impl/matrix-ops.lisp:10-15``), the column sums the AddNode of the bias sends back, and the
    backward of unfold.  ``col`` is recomputed (the reference saves it)."""
    stride, padding = _pair(stride), _pair(padding)
    N, _, H, W = x.shape
    c_out, c_in, kh, kw = weight.shape
    col = F.unfold(x, (1, 1), (kh, kw), stride, padding)                 # [(N h w) (C k-h k-w)]
    dy = F.reshape(dout.permute(0, 2, 3, 1), -1, c_out)                  # [(N h w) C_out], a copy
    col_w = F.reshape(weight, c_out, -1)
    dweight = F.reshape(F.matmul(F.t(dy), col), c_out, c_in, kh, kw)
    dbias = F.sum(dy, axis=0) if bias else None
    dcol = F.matmul(dy, col_w)
    return F.unfold_backward(dcol, x.shape, (kh, kw), stride, padding), dweight, dbias


def _pool_backward(x: HIPTensor, dout: HIPTensor, kernel_size, stride, padding, spread) -> HIPTensor:
    kernel_size, stride, padding = _pair(kernel_size), _pair(stride), _pair(padding)
    N, Cc, H, W = x.shape
    k = kernel_size[0] * kernel_size[1]
    windows = F.reshape(F.unfold(x, (1, 1), kernel_size, stride, padding), -1, k)   # [(N h w C) (k-h k-w)]
    d = F.reshape(dout.permute(0, 2, 3, 1), -1, 1)                                    # [(N h w C) 1], a copy
    dwin = spread(windows, d.view(True, (":broadcast", k)))
    return F.unfold_backward(F.reshape(dwin, -1, Cc * k), x.shape, kernel_size, stride, padding)


def max_pool2d_backward(x: HIPTensor, dout: HIPTensor, kernel_size, stride=None, padding=0) -> HIPTensor:
    """The gradient of :func:`max_pool2d`: MaxValue-Node sends ``dout`` to every element of a window that
    equals its maximum (the mask ``A=B a max(a)``, ``base-impl/matrix-ops.lisp:312-334``), unfold's backward
    folds the windows."""
    def spread(windows, d):
        top = F.max(windows, axis=1, keepdims=True)
        return F.mul_(F.compare(windows, top, "="), d)
    return _pool_backward(x, dout, kernel_size, kernel_size if stride is None else stride, padding, spread)


def avg_pool2d_backward(x: HIPTensor, dout: HIPTensor, kernel_size, stride=None, padding=0) -> HIPTensor:
    """The gradient of :func:`avg_pool2d`: ``dout / (k-h k-w)`` to every element of the window."""
    k = _pair(kernel_size)
    def spread(windows, d):
        return F.div_(F.copy(d), float(k[0] * k[1]))
    return _pool_backward(x, dout, kernel_size, kernel_size if stride is None else stride, padding, spread)


# ---------------------------------------------------------------------------
# criteria (source/nn/criterion.lisp), composed from the backend's nodes
# ---------------------------------------------------------------------------

def _reduce(z: HIPTensor, reduction):
    if reduction == "sum":
        return F.sum(z)
    if reduction == "mean":
        return F.mean(z)
    return z


def mse(x: HIPTensor, y: HIPTensor, reduction="mean") -> HIPTensor:
    """``(mse x y :reduction :mean)`` (criterion.lisp:48-80): ``(x - y)^2``."""
    l = F.sub(x, y)
    return _reduce(F.mul(l, l), reduction)


def cross_entropy_loss(x: HIPTensor, labels: HIPTensor, delta: float = 1e-7, reduction=True) -> HIPTensor:
    """``(cross-entropy-loss x labels :delta 1e-7)`` (criterion.lisp:128-167):
    ``-labels * log(x + delta)`` with one-hot ``labels``."""
    z = F.mul(F.mul(labels, F.loge(F.add(x, delta))), -1.0)
    return _reduce(z, reduction)


def softmax_cross_entropy(x: HIPTensor, labels: HIPTensor, axis: int = 1, delta: float = 1e-7,
                          avoid_overflow: bool = False, reduction=True):
    """``(softmax-cross-entropy x labels ...)`` = Softmax-Cross-Entropy-Node
    (criterion.lisp:90-126,169-196): softmax, then the cross entropy.  Returns
    ``(loss, z)`` where ``z`` is the softmax the node saves for its backward."""
    z = F.softmax(x, avoid_overflow=avoid_overflow, axis=axis)
    return _reduce(cross_entropy_loss(z, labels, delta=delta), reduction), z


def softmax_cross_entropy_backward(dy, z: HIPTensor, labels: HIPTensor) -> HIPTensor:
    """The node's backward, ``sce-diff-static`` (criterion.lisp:82-88):
    ``dy * (z - labels) / batch`` with ``batch`` the second-to-last extent of
    ``z``; ``dy`` is the upstream gradient (a tensor of z's shape or a number)."""
    batch = float(z.shape[-2])
    return F.div(F.mul(F.sub(z, labels), dy), batch)


def softmax_cross_entropy_fused(x: HIPTensor, labels: HIPTensor, delta: float = 1e-7, reduction=True):
    """``(softmax-cross-entropy x labels)`` with the classes on the last axis as ONE node
    (HIP-Softmax-Cross-Entropy-Node; ``softmax-cross-entropy-hip`` of the Lisp glue): the softmax is
    max-subtracted (the kernel of HIP-Softmax-Node) where !softmax subtracts the mean or nothing, the
    cross entropy rounds like the reference's nodes.  Returns ``(loss, z)`` like
    :func:`softmax_cross_entropy`."""
    x, labels = F.to_contiguous(x), F.to_contiguous(labels)
    z = HIPTensor(list(x.shape), initial_element=None)
    out = HIPTensor(list(x.shape), initial_element=None)
    nodes.forward("HIP-Softmax-Cross-Entropy-Node", x, labels, z, out, float(delta))
    return _reduce(out, reduction), z


def softmax_cross_entropy_backward_fused(dy, z: HIPTensor, labels: HIPTensor, in_place: bool = False) -> HIPTensor:
    """:func:`softmax_cross_entropy_backward` as ONE node (HIP-Softmax-Cross-Entropy-Node-backward), bit for
    bit the same result.  ``dy``: a tensor of z's shape, a one-element tensor or a number.  With
    ``in_place`` the gradient overwrites a full-shape ``dy``."""
    if not isinstance(dy, HIPTensor):
        dy = HIPTensor([1], initial_element=float(dy))
    dy, labels = F.to_contiguous(dy), F.to_contiguous(labels)
    full = list(dy.shape) == list(z.shape)
    dx = dy if (in_place and full) else HIPTensor(list(z.shape), initial_element=None)
    return nodes.forward("HIP-Softmax-Cross-Entropy-Node-backward", dy, z, labels, dx)
