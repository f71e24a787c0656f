"""Softmax-Cross-Entropy-Node as one kernel forward and one backward (source/nn/criterion.lisp:82-126):
against a float64 closed form of the node, against the node compositions (bit for bit where the
arithmetic is the same), and inside a training loop.

The reference holds no vectors for this node (its tests run it on random (10, 10) tensors and check
that it runs and that the gradient is not all zero, source/nn/t/criterion.lisp:3-31), so the float64
closed form below, pinned by the identities it is tested with, is the checker: parity unpinned by the
reference."""
import numpy as np
import pytest

from helpers import assert_bit_equal

pytestmark = pytest.mark.gpu
f32 = np.float32
DELTA = 1e-7


def _truth(x, labels, delta=DELTA):
    """float64: z = softmax over the last axis, loss = -labels log(z + delta) with delta the binary32 number
    the node holds."""
    x = x.astype(np.float64)
    e = np.exp(x - x.max(axis=-1, keepdims=True))
    z = e / e.sum(axis=-1, keepdims=True)
    return z, -labels.astype(np.float64) * np.log(z + np.float64(f32(delta)))


def _labels(rng, rows, cols, kind):
    if kind == "one-hot":
        return np.eye(cols, dtype=f32)[rng.integers(0, cols, rows)]
    t = rng.random((rows, cols)).astype(f32) ** 4
    return (t / t.sum(axis=1, keepdims=True)).astype(f32)


def test_truth_identities():
    """What pins the closed form: rows of z sum to 1; with one-hot labels the summed loss is
    logsumexp(x) - x[class] (delta = 0); the gradient of the mean loss is (z - labels) / count by
    central differences."""
    rng = np.random.default_rng(5)
    x = rng.standard_normal((6, 11)) * 3
    cls = rng.integers(0, 11, 6)
    t = np.eye(11)[cls]
    z, loss = _truth(x, t, delta=0.0)
    assert np.allclose(z.sum(axis=1), 1.0, atol=1e-14)
    lse = np.log(np.exp(x).sum(axis=1))
    assert np.allclose(loss.sum(axis=1), lse - x[np.arange(6), cls], atol=1e-12)
    g = (z - t) / x.size
    h = 1e-6
    for (i, j) in [(0, 0), (2, 5), (5, 10), (3, int(cls[3]))]:
        xp, xm = x.copy(), x.copy()
        xp[i, j] += h
        xm[i, j] -= h
        num = (_truth(xp, t, 0.0)[1].mean() - _truth(xm, t, 0.0)[1].mean()) / (2 * h)
        assert abs(num - g[i, j]) <= 1e-9


# every row form of the kernel: four rows per wavefront (256 columns and fewer), two (512), one (768 ... 4096,
# 1024 as two wavefronts per row), a workgroup of 1024 threads per row up to 65536 columns (2, 4, 8, 13, 16
# vectors per thread), three passes beyond; row counts that leave ragged last workgroups; from 16384 rows of at
# most 64 columns on, a thread per row
SHAPES = [(20001, 10), (16390, 33), (16384, 64), (16384, 32), (16390, 1), (17000, 31), (40000, 4), (100, 10), (7, 3), (1, 1), (257, 256), (65, 500), (33, 768), (101, 1000), (64, 1024), (9, 1537),
          (11, 2048), (6, 3072), (5, 4096), (4, 5000), (3, 50257), (5, 8192), (4, 8197), (3, 20000), (3, 32768),
          (3, 60000), (3, 66000),
          # at least a row per compute unit: a workgroup per row up to 65536 columns, rows off a 16-byte boundary
          (260, 8195), (257, 20001), (258, 40001), (257, 50257), (256, 65536)]


@pytest.mark.parametrize("rows,cols", SHAPES)
@pytest.mark.parametrize("kind", ["one-hot", "soft"])
def test_forward(gpu, rows, cols, kind):
    W = gpu
    F, nn = W.functional, W.nn
    rng = np.random.default_rng(rows * 7919 + cols)
    x = (rng.standard_normal((rows, cols)) * 4).astype(f32)
    if rows > 2:
        x[1] = x[1] * 30          # a row whose small probabilities underflow: loss = -label log(delta) there
        x[2, : cols // 2 + 1] = -np.inf if cols > 1 else x[2, 0]
    t = _labels(rng, rows, cols, kind)
    dx, dt = F.from_numpy(x), F.from_numpy(t)
    loss, z = nn.softmax_cross_entropy_fused(dx, dt, delta=DELTA, reduction=True)
    got_z, got_loss = z.numpy(), loss.numpy()
    # the softmax is the kernel of HIP-Softmax-Node, the cross entropy the reference's nodes
    assert_bit_equal(got_z, F.softmax_fused(dx).numpy(), "z against HIP-Softmax-Node")
    assert_bit_equal(got_loss, nn.cross_entropy_loss(z, dt, delta=DELTA, reduction=True).numpy(),
                     "loss against the nodes of cross-entropy-loss")
    assert_bit_equal(dx.numpy(), x, "x untouched")
    assert_bit_equal(dt.numpy(), t, "labels untouched")
    want_z, want_loss = _truth(x, t)
    # exp(d) carries the rounding of d = x - max (|d| 2^-24 relative); below the normal numbers the
    # exponential instruction returns 0
    assert np.all(np.abs(got_z - want_z) <= 8e-6 * want_z + 1.2e-38)
    # log(z + delta): the argument carries z's error (relative, a few 2^-24, plus the rounding of the sum),
    # the logarithm its own ulp
    bar = np.abs(t.astype(np.float64)) * (4e-6 + 2.0 ** -22 * np.abs(np.log(want_z + DELTA))) + 1e-30
    assert np.max(np.abs(got_loss - want_loss) / bar) <= 1.0


def test_forward_reductions_and_delta(gpu):
    W = gpu
    F, nn = W.functional, W.nn
    rng = np.random.default_rng(8)
    x = (rng.standard_normal((128, 10)) * 2).astype(f32)
    t = _labels(rng, 128, 10, "one-hot")
    for delta in (1e-7, 1e-3, 0.0):
        want = _truth(x, t, delta)[1]
        for reduction, ref in (("sum", want.sum()), ("mean", want.mean())):
            loss, _ = nn.softmax_cross_entropy_fused(F.from_numpy(x), F.from_numpy(t), delta=delta, reduction=reduction)
            assert abs(float(loss.numpy().ravel()[0]) - ref) <= 2e-6 * abs(ref)
    # the composed node of the reference's recipe (mean-subtracted softmax) lands on the same loss
    comp, _ = nn.softmax_cross_entropy(F.from_numpy(x), F.from_numpy(t), avoid_overflow=True, reduction="mean")
    one, _ = nn.softmax_cross_entropy_fused(F.from_numpy(x), F.from_numpy(t), reduction="mean")
    assert abs(float(comp.numpy().ravel()[0]) - float(one.numpy().ravel()[0])) <= 2e-6 * abs(float(one.numpy().ravel()[0]))


def test_forward_views_are_materialised(gpu):
    """Transposed logits and a window of a wider label tensor: the wrapper hands contiguous copies down."""
    W = gpu
    F, nn = W.functional, W.nn
    rng = np.random.default_rng(9)
    xt = (rng.standard_normal((40, 24)) * 2).astype(f32)
    wide = rng.random((24, 100)).astype(f32)
    loss, z = nn.softmax_cross_entropy_fused(F.from_numpy(xt).permute(1, 0), F.from_numpy(wide).view(True, (30, 70)))
    want_z, want = _truth(xt.T, wide[:, 30:70])
    assert np.max(np.abs(z.numpy() - want_z)) <= 1e-6
    assert np.max(np.abs(loss.numpy() - want)) <= 1e-5 * np.max(np.abs(want))


@pytest.mark.parametrize("shape", [(100, 10), (7, 3), (33, 1000), (3, 5, 64), (4097, 1023), (16384, 1024)])
def test_backward(gpu, shape):
    """(dy (z - labels)) / batch: the bits of the SubNode, MulNode and DivNode of sce-diff-static, for a
    gradient tensor, for one number and in place; (16384, 1024) takes the streaming loads."""
    W = gpu
    F, nn = W.functional, W.nn
    rng = np.random.default_rng(len(shape) * 31 + shape[-1])
    z = rng.random(shape).astype(f32)
    t = _labels(rng, int(np.prod(shape[:-1])), shape[-1], "one-hot").reshape(shape)
    dy = rng.standard_normal(shape).astype(f32)
    dz, dt, ddy = F.from_numpy(z), F.from_numpy(t), F.from_numpy(dy)
    want = nn.softmax_cross_entropy_backward(ddy, dz, dt).numpy()
    got = nn.softmax_cross_entropy_backward_fused(ddy, dz, dt).numpy()
    assert_bit_equal(got, want, "tensor gradient against the nodes")
    batch = float(shape[-2])
    truth = dy.astype(np.float64) * (z.astype(np.float64) - t) / batch
    assert np.max(np.abs(got - truth)) <= 3 * 2.0 ** -24 * np.max(np.abs(truth)) + 1e-30
    assert_bit_equal(ddy.numpy(), dy, "dy untouched when not in place")
    # one number for every element
    s = 1.0 / z.size
    assert_bit_equal(nn.softmax_cross_entropy_backward_fused(s, dz, dt).numpy(),
                     nn.softmax_cross_entropy_backward(s, dz, dt).numpy(), "scalar gradient against the nodes")
    one = F.from_numpy(np.array([s], f32))
    assert_bit_equal(nn.softmax_cross_entropy_backward_fused(one, dz, dt).numpy(),
                     nn.softmax_cross_entropy_backward(s, dz, dt).numpy(), "one-element gradient tensor")
    # in place
    out = nn.softmax_cross_entropy_backward_fused(ddy, dz, dt, in_place=True)
    assert out is ddy
    assert_bit_equal(ddy.numpy(), want, "in place")
    assert_bit_equal(dz.numpy(), z, "z untouched")


def test_backward_unaligned_storage(gpu):
    """Tensors that start 4 bytes into an allocation take the scalar path: same bits."""
    W = gpu
    F = W.functional
    import ctypes as C
    rng = np.random.default_rng(12)
    n = 1003
    z, t, dy = (rng.random(n + 1).astype(f32) for _ in range(3))
    bufs = [F.from_numpy(a) for a in (dy, z, t)]
    dx = W.HIPTensor([n + 1])
    lib = W.lib.get()
    W.lib.check(lib.wf2hip_softmax_cross_entropy_backward_f32(n, C.c_void_p(bufs[0].ptr + 4), 0, C.c_void_p(bufs[1].ptr + 4),
                                                              C.c_void_p(bufs[2].ptr + 4), 7.0, C.c_void_p(dx.ptr + 4)))
    want = (dy[1:] * (z[1:] - t[1:])) / f32(7.0)
    assert_bit_equal(dx.numpy()[1:], want, "offset storage")
    assert dx.numpy()[0] == 0.0


def test_argument_checks(gpu):
    W = gpu
    F = W.functional
    import ctypes as C
    lib = W.lib.get()
    a, b, c, d = (W.HIPTensor([8, 16]) for _ in range(4))
    p = lambda t: C.c_void_p(t.ptr)  # noqa: E731
    assert lib.wf2hip_softmax_cross_entropy_f32(8, 16, p(a), p(b), 1e-7, p(a), p(d)) == W.lib.EOVERLAP   # z is x
    assert lib.wf2hip_softmax_cross_entropy_f32(8, 16, p(a), p(b), 1e-7, p(c), p(c)) == W.lib.EOVERLAP   # loss is z
    assert lib.wf2hip_softmax_cross_entropy_f32(8, 16, p(a), p(b), 1e-7, p(c), p(b)) == W.lib.EOVERLAP   # loss is labels
    assert lib.wf2hip_softmax_cross_entropy_f32(8, 16, p(a), None, 1e-7, p(c), p(d)) == W.lib.EINVAL
    assert lib.wf2hip_softmax_cross_entropy_f32(-1, 16, p(a), p(b), 1e-7, p(c), p(d)) == W.lib.EINVAL
    assert lib.wf2hip_softmax_cross_entropy_f32(0, 16, p(a), p(b), 1e-7, p(c), p(d)) == 0
    bw = lib.wf2hip_softmax_cross_entropy_backward_f32
    assert bw(128, p(a), 0, p(b), p(c), 8.0, p(c)) == W.lib.EOVERLAP          # dx is labels
    assert bw(128, p(a), 0, p(b), p(c), 8.0, C.c_void_p(b.ptr + 16)) == W.lib.EOVERLAP   # dx meets z, shifted
    assert bw(128, p(a), 1, p(b), p(c), 8.0, p(a)) == W.lib.EOVERLAP          # dx covers the one number it reads
    assert bw(128, p(a), 0, p(b), p(c), 8.0, p(b)) == 0                       # dx is z
    assert bw(128, None, 0, p(b), p(c), 8.0, p(d)) == W.lib.EINVAL
    assert bw(0, p(a), 0, p(b), p(c), 8.0, p(d)) == 0
    with pytest.raises(ValueError):
        W.nodes.forward("HIP-Softmax-Cross-Entropy-Node", a, W.HIPTensor([8, 15]), c, d)
    with pytest.raises(ValueError):
        W.nodes.forward("HIP-Softmax-Cross-Entropy-Node-backward", W.HIPTensor([3]), b, c, d)
    del F
