"""Im2ColNode / Col2ImNode kernels: bitwise against the oracle (pinned to the
reference's compiled im2col.c by tests/test_oracle_golden.py) and against the
golden outputs themselves; the adjoint identity at a larger size; `unfold`
against the sliding-window closed form."""
import ctypes as C
import importlib.util
import os

import numpy as np
import pytest

from helpers import assert_bit_equal

pytestmark = pytest.mark.gpu
HERE = os.path.dirname(os.path.abspath(__file__))


def _golden_module():
    spec = importlib.util.spec_from_file_location("make_golden", os.path.join(HERE, "golden", "make_golden.py"))
    mg = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mg)
    return mg


def test_im2col_col2im_golden(gpu):
    W = gpu
    mg = _golden_module()
    gold = np.load(os.path.join(HERE, "golden", "im2col_kernels.npz"))
    for idx, case in enumerate(mg.IM2COL_CASES):
        N, Cc, H, Wd, Ho, Wo, kh, kw = mg.im2col_geometry(case)
        _, _, _, _, k, s, p = case
        x = W.HIPTensor.from_numpy(gold[f"im2col_{idx}_im"])
        col = W.HIPTensor.from_numpy(np.full((N, Cc, kh, kw, Ho, Wo), 7.0, np.float32))
        W.forward("Im2ColNode", x, col, s, p, (1, 1))
        assert_bit_equal(col.numpy(), gold[f"im2col_{idx}_col"], f"im2col case {idx}")
        back = W.HIPTensor.from_numpy(np.full((N, Cc, H, Wd), 5.0, np.float32))
        W.forward("Col2ImNode", W.HIPTensor.from_numpy(gold[f"col2im_{idx}_col"]), back, s, p, (1, 1))
        assert_bit_equal(back.numpy(), gold[f"col2im_{idx}_im"], f"col2im case {idx}")


@pytest.mark.parametrize("seed", range(6))
def test_im2col_random_geometries_match_oracle(gpu, O, seed):
    """Kernels of 1 ... 7 rows and columns (square ones of 1, 2, 3, 5 and 7 take unrolled loops in
    col2im, the others the loops over the extents), strides 1 ... 3, padding 0 ... 2; the later
    seeds draw images of several workgroups."""
    W = gpu
    rng = np.random.default_rng(40 + seed)
    top = 20 if seed < 3 else 45
    for case in range(10):
        N, Cc = int(rng.integers(1, 4)), int(rng.integers(1, 5))
        k = (int(rng.integers(1, 8)), int(rng.integers(1, 8)))
        if case % 2:
            k = (k[0], k[0])
        s = (int(rng.integers(1, 4)), int(rng.integers(1, 4)))
        p = (int(rng.integers(0, 3)), int(rng.integers(0, 3)))
        Hin, Win = int(rng.integers(k[0], top)), int(rng.integers(k[1], top))
        out = [(size + 2 * p[a] - (k[a] - 1) - 1) // s[a] + 1 for a, size in enumerate((Hin, Win))]
        H, Wd = [size + 2 * p[a] + out[a] % s[a] for a, size in enumerate((Hin, Win))]
        im = rng.standard_normal((N, Cc, H, Wd)).astype(np.float32)
        start = rng.standard_normal((N, Cc, k[0], k[1], out[0], out[1])).astype(np.float32)
        want = start.copy()  # what the walk does not reach keeps the value it held
        O.im2col(want, im, N, Cc, H, Wd, out[0], out[1], k[0], k[1], p, s, (1, 1))
        col = W.HIPTensor.from_numpy(start)
        W.forward("Im2ColNode", W.HIPTensor.from_numpy(im), col, s, p, (1, 1))
        assert_bit_equal(col.numpy(), want, f"im2col {N, Cc, H, Wd, k, s, p}")
        cin = rng.standard_normal(want.shape).astype(np.float32)
        want_im = np.zeros_like(im)
        O.col2im(cin, want_im, N, Cc, H, Wd, out[0], out[1], k[0], k[1], p, s, (1, 1))
        back = W.HIPTensor([N, Cc, H, Wd])
        W.forward("Col2ImNode", W.HIPTensor.from_numpy(cin), back, s, p, (1, 1))
        assert_bit_equal(back.numpy(), want_im, f"col2im {N, Cc, H, Wd, k, s, p}")


@pytest.mark.parametrize("N,Cc,Hin,Win,k,s,p", [
    (2, 3, 130, 200, (3, 3), (1, 1), (1, 1)),     # several bands of rows per image plane
    (1, 2, 40, 5000, (3, 3), (1, 1), (0, 0)),     # rows too wide for the staged kernel
    (1, 2, 9, 3000, (5, 2), (1, 1), (2, 0)),      # the larger tile
    (2, 2, 64, 64, (2, 2), (2, 2), (0, 0)),       # pooling windows: no overlap, strides powers of two
    (2, 2, 63, 66, (3, 3), (3, 3), (0, 0)),       # no overlap, stride 3
    (2, 2, 61, 67, (2, 3), (3, 4), (1, 1)),       # kernel smaller than the stride
    (3, 2, 57, 57, (3, 3), (2, 2), (1, 1)),       # overlap with stride 2
    (1, 1, 300, 300, (7, 7), (2, 2), (3, 3)),
    (3, 5, 56, 56, (3, 3), (1, 1), (1, 1)),       # one band per plane, one element short at the end of every row
    (2, 3, 60, 64, (3, 5), (1, 1), (2, 2)),       # two elements short
    (2, 2, 120, 98, (5, 5), (1, 1), (1, 3)),      # several bands, three short
    (8, 64, 56, 56, (3, 3), (1, 1), (1, 1)),      # a whole plane per workgroup, the old values staged
    (8, 64, 28, 28, (5, 5), (1, 1), (1, 3)),      # more old values than a workgroup stages: single stores around them
])
def test_im2col_larger_geometries_match_oracle(gpu, O, N, Cc, Hin, Win, k, s, p):
    """Each dispatch of the two kernels at sizes of many workgroups, bit for bit against the compiled
    restatement of the reference's loops (elements its walk does not reach keep the values they held)."""
    W = gpu
    rng = np.random.default_rng(Hin * 1000 + Win)
    out = [(size + 2 * p[a] - (k[a] - 1) - 1) // s[a] + 1 for a, size in enumerate((Hin, Win))]
    H, Wd = [size + 2 * p[a] + out[a] % s[a] for a, size in enumerate((Hin, Win))]
    im = rng.standard_normal((N, Cc, H, Wd)).astype(np.float32)
    start = rng.standard_normal((N, Cc, k[0], k[1], out[0], out[1])).astype(np.float32)
    want = start.copy()
    O.im2col(want, im, N, Cc, H, Wd, out[0], out[1], k[0], k[1], p, s, (1, 1))
    col = W.HIPTensor.from_numpy(start)
    W.forward("Im2ColNode", W.HIPTensor.from_numpy(im), col, s, p, (1, 1))
    assert_bit_equal(col.numpy(), want, "im2col")
    cin = rng.standard_normal(want.shape).astype(np.float32)
    want_im = np.zeros_like(im)
    O.col2im(cin, want_im, N, Cc, H, Wd, out[0], out[1], k[0], k[1], p, s, (1, 1))
    back = W.HIPTensor.from_numpy(np.full(im.shape, 9.0, np.float32))
    W.forward("Col2ImNode", W.HIPTensor.from_numpy(cin), back, s, p, (1, 1))
    assert_bit_equal(back.numpy(), want_im, "col2im")


def test_unfold_and_adjoint(gpu):
    """unfold(x) for stride 1 without padding is the sliding window of numpy,
    laid out [(N h-out w-out) (C k-h k-w)]; at a convolution-sized input
    <im2col(x), c> = <x, col2im(c)> (the two kernels are adjoint)."""
    W = gpu
    F = W.functional
    rng = np.random.default_rng(8)
    x = rng.standard_normal((2, 3, 9, 8)).astype(np.float32)
    got = F.unfold(F.from_numpy(x), (1, 1), (3, 2), (1, 1), (0, 0)).numpy()
    win = np.lib.stride_tricks.sliding_window_view(x, (3, 2), axis=(2, 3))     # N C ho wo kh kw
    want = win.transpose(0, 2, 3, 1, 4, 5).reshape(2 * 7 * 7, 3 * 3 * 2)
    assert_bit_equal(got, np.ascontiguousarray(want), "unfold")
    N, Cc, H, Wd, k, s = 8, 16, 66, 66, (3, 3), (1, 1)
    Ho, Wo = H - 2, Wd - 2
    xi = rng.standard_normal((N, Cc, H, Wd)).astype(np.float32)
    ci = rng.standard_normal((N, Cc, 3, 3, Ho, Wo)).astype(np.float32)
    col = W.HIPTensor([N, Cc, 3, 3, Ho, Wo])
    W.forward("Im2ColNode", F.from_numpy(xi), col, s, (0, 0), (1, 1))
    back = W.HIPTensor([N, Cc, H, Wd])
    W.forward("Col2ImNode", F.from_numpy(ci), back, s, (0, 0), (1, 1))
    lhs = np.sum(col.numpy().astype(np.float64) * ci)
    rhs = np.sum(xi.astype(np.float64) * back.numpy())
    assert abs(lhs - rhs) <= 1e-6 * np.sum(np.abs(xi)) 


def test_im2col_argument_checks(gpu):
    W = gpu
    lib = W.lib.get()
    a = W.HIPTensor([1, 1, 8, 8])
    col = W.HIPTensor([1, 1, 3, 3, 6, 6])
    args = lambda **kw: [kw.get(n, d) for n, d in (("N", 1), ("C", 1), ("H", 8), ("W", 8), ("Ho", 6), ("Wo", 6), ("kh", 3),  # noqa: E731
                                                   ("kw", 3), ("ph", 0), ("pw", 0), ("sh", 1), ("sw", 1), ("dh", 1), ("dw", 1))]
    c, x = C.c_void_p(col.ptr), C.c_void_p(a.ptr)
    assert lib.wf2hip_im2col_f32(c, *args(), x) == 0
    assert lib.wf2hip_im2col_f32(c, *args(dh=2), x) == -4          # the walk would leave its plane
    assert lib.wf2hip_im2col_f32(c, *args(H=7), x) == -1           # the walk leaves the image
    assert lib.wf2hip_im2col_f32(c, *args(sh=0), x) == -1
    assert lib.wf2hip_col2im_f32(c, *args(kh=40), x) == -4


def test_reference_unfold_vectors(gpu):
    """source/nn/t/conv.lisp:41-56: unfold of (ax+b (2 2 2 2) 1 0) with a 2x2
    kernel is 0..15, and the backward of sum(out * (ax+b (2 8) 1 0)) through
    Col2ImNode is 0..15 again; Conv2D 3 -> 6, 2x2 on (3 3 10 10) gives (3 6 9 9)
    (:6)."""
    W = gpu
    F = W.functional
    img = F.from_numpy(np.arange(16, dtype=np.float32).reshape(2, 2, 2, 2))
    out = F.unfold(img, (1, 1), (2, 2), (1, 1), (0, 0))
    assert out.shape == [2, 8]
    assert np.array_equal(out.numpy().ravel(), np.arange(16, dtype=np.float32))
    # d/d img of sum(out * g): g laid back as Col[N C kh kw 1 1], folded by Col2ImNode
    g = np.arange(16, dtype=np.float32).reshape(2, 1, 1, 2, 2, 2).transpose(0, 3, 4, 5, 1, 2)
    back = W.HIPTensor([2, 2, 2, 2])
    W.forward("Col2ImNode", F.from_numpy(np.ascontiguousarray(g)), back, (1, 1), (0, 0), (1, 1))
    assert np.array_equal(back.numpy().ravel(), np.arange(16, dtype=np.float32))
    rng = np.random.default_rng(0)
    y = W.nn.conv2d(F.from_numpy(rng.standard_normal((3, 3, 10, 10)).astype(np.float32)),
                    F.from_numpy(rng.standard_normal((6, 3, 2, 2)).astype(np.float32)),
                    F.from_numpy(rng.standard_normal(6).astype(np.float32)))
    assert y.shape == [3, 6, 9, 9]


@pytest.mark.parametrize("stride", [1, 2])
def test_conv_and_pooling_layers(gpu, stride):
    """Conv2D / MaxPool2D / AvgPool2D composed from the nodes, against float64
    closed forms (no padding: with padding the reference's walk leaves the last
    rows of Col untouched, which the im2col tests above pin instead)."""
    W = gpu
    F = W.functional
    rng = np.random.default_rng(stride)
    x = rng.standard_normal((2, 3, 12, 11)).astype(np.float32)
    w = rng.standard_normal((5, 3, 3, 2)).astype(np.float32)
    b = rng.standard_normal(5).astype(np.float32)
    y = W.nn.conv2d(F.from_numpy(x), F.from_numpy(w), F.from_numpy(b), stride=stride).numpy()
    win = np.lib.stride_tricks.sliding_window_view(x.astype(np.float64), (3, 2), axis=(2, 3))[:, :, ::stride, ::stride]
    want = np.einsum("nchwij,ocij->nohw", win, w.astype(np.float64)) + b[None, :, None, None]
    np.testing.assert_allclose(y, want, rtol=1e-5, atol=1e-5)
    pw = np.lib.stride_tricks.sliding_window_view(x, (2, 2), axis=(2, 3))[:, :, ::2, ::2]
    assert_bit_equal(W.nn.max_pool2d(F.from_numpy(x), 2).numpy(), pw.max(axis=(4, 5)), "max pool")
    np.testing.assert_allclose(W.nn.avg_pool2d(F.from_numpy(x), 2).numpy(),
                               pw.astype(np.float64).mean(axis=(4, 5)), rtol=1e-6, atol=1e-6)


UNFOLD_CASES = [
    # N, C, H, W, kernel, stride, padding
    (2, 3, 12, 11, (3, 2), (1, 1), (0, 0)),
    (2, 3, 12, 11, (3, 3), (1, 1), (1, 1)),      # padded: the walk leaves the last row and column of every plane at 0
    (3, 5, 17, 19, (3, 3), (2, 2), (1, 1)),
    (2, 4, 16, 16, (2, 2), (2, 2), (0, 0)),      # pooling windows
    (1, 1, 28, 28, (5, 5), (1, 1), (2, 2)),
    (2, 2, 9, 40, (1, 1), (1, 1), (0, 0)),
    (2, 70, 20, 20, (3, 3), (1, 1), (1, 1)),     # channels in chunks, the last one short
    (1, 3, 70, 300, (3, 3), (1, 1), (1, 1)),     # rows wider than a band of 256 positions
    (1, 2, 33, 31, (7, 7), (3, 2), (3, 3)),
    (2, 3, 15, 14, (4, 3), (3, 4), (2, 1)),      # kernel smaller than the stride along W
    (4, 64, 56, 56, (3, 3), (1, 1), (1, 1)),     # a ResNet-style layer
    (1, 2, 6, 2200, (3, 3), (1, 1), (0, 0)),     # one channel of one output row needs more than the first budget
]


@pytest.mark.parametrize("N,Cc,H,Wd,k,s,p", UNFOLD_CASES)
def test_unfold_as_one_node_is_the_composition(gpu, N, Cc, H, Wd, k, s, p):
    """HIP-Unfold-Node against the node composition of unfold (padding, Im2ColNode into a zeroed col,
    permutation, reshape), which the reference's vectors and the compiled im2col pin: pure data
    movement, so bit for bit, -0.0 and NaN included."""
    W = gpu
    F = W.functional
    rng = np.random.default_rng(H * 131 + Wd)
    x = rng.standard_normal((N, Cc, H, Wd)).astype(np.float32)
    x.flat[:3] = [-0.0, np.nan, np.inf]
    dx = F.from_numpy(x)
    want = F.unfold_composed(dx, (1, 1), k, s, p).numpy()
    out = F.unfold(dx, (1, 1), k, s, p)
    assert out.shape == list(want.shape)
    assert_bit_equal(out.numpy(), want, "unfold")
    assert_bit_equal(dx.numpy(), x, "x untouched")


def test_unfold_node_arguments_and_fallback(gpu):
    W = gpu
    F = W.functional
    import ctypes as C
    lib = W.lib.get()
    x = W.HIPTensor([1, 1, 4, 4])
    out = W.HIPTensor([9, 4])
    ptr = lambda t: C.c_void_p(t.ptr)  # noqa: E731
    assert lib.wf2hip_unfold_f32(1, 1, 4, 4, 2, 2, 1, 1, 0, 0, ptr(x), ptr(out)) == 0
    assert lib.wf2hip_unfold_f32(1, 1, 4, 4, 5, 2, 1, 1, 0, 0, ptr(x), ptr(out)) == W.lib.EINVAL    # kernel taller than the image
    assert lib.wf2hip_unfold_f32(1, 1, 4, 4, 2, 2, 0, 1, 0, 0, ptr(x), ptr(out)) == W.lib.EINVAL
    assert lib.wf2hip_unfold_f32(1, 1, 4, 4, 2, 2, 1, 1, 0, 0, ptr(x), None) == W.lib.EINVAL
    assert lib.wf2hip_unfold_f32(1, 1, 4, 4, 2, 2, 1, 1, 0, 0, ptr(x), ptr(x)) == W.lib.EOVERLAP
    assert lib.wf2hip_unfold_f32(0, 1, 4, 4, 2, 2, 1, 1, 0, 0, ptr(x), ptr(out)) == 0
    with pytest.raises(ValueError):
        W.forward("HIP-Unfold-Node", x, W.HIPTensor([9, 5]), (2, 2), (1, 1), (0, 0))
    # a row too wide for the kernel's staging memory: the library refuses, unfold composes
    wide = F.from_numpy(np.random.default_rng(1).standard_normal((1, 1, 3, 20000)).astype(np.float32))
    tall_out = W.HIPTensor([19998, 9])
    assert lib.wf2hip_unfold_f32(1, 1, 3, 20000, 3, 3, 1, 1, 0, 0, ptr(wide), ptr(tall_out)) == W.lib.EUNSUPPORTED
    assert_bit_equal(F.unfold(wide, (1, 1), (3, 3), (1, 1), (0, 0)).numpy(),
                     F.unfold_composed(wide, (1, 1), (3, 3), (1, 1), (0, 0)).numpy(), "fallback")


@pytest.mark.parametrize("N,Cc,H,Wd,k,s,p", UNFOLD_CASES[:10])
def test_unfold_backward_is_the_adjoint(gpu, N, Cc, H, Wd, k, s, p):
    """<unfold(x), c> = <x, unfold_backward(c)> where the walk reaches every position (no padding), and in
    general unfold_backward(c) is the float64 gradient of sum(unfold(x) * c) by its definition: each
    element of x collects the c of the matrix entries that hold it."""
    W = gpu
    F = W.functional
    rng = np.random.default_rng(H * 7 + Wd)
    x = rng.standard_normal((N, Cc, H, Wd)).astype(np.float32)
    col = F.unfold(F.from_numpy(x), (1, 1), k, s, p).numpy()
    c = rng.standard_normal(col.shape).astype(np.float32)
    back = F.unfold_backward(F.from_numpy(c), x.shape, k, s, p).numpy()
    assert back.shape == x.shape
    # the matrix entries as a linear map of x: push an index image through the same unfold
    idx = np.arange(1, x.size + 1, dtype=np.float32).reshape(x.shape)       # exact below 2^24
    assert x.size < 2 ** 24
    where = F.unfold(F.from_numpy(idx), (1, 1), k, s, p).numpy().astype(np.int64)   # 0: padding or not reached
    want = np.zeros(x.size + 1, np.float64)
    np.add.at(want, where.ravel(), c.astype(np.float64).ravel())
    want = want[1:].reshape(x.shape)
    mag = np.zeros(x.size + 1, np.float64)
    np.add.at(mag, where.ravel(), np.abs(c).astype(np.float64).ravel())
    assert np.all(np.abs(back - want) <= 1e-6 * mag[1:].reshape(x.shape) + 1e-30)
