"""GPU parity of the element-wise kernels against the CPU oracle.

Bar: bit-exact for add/sub/mul/div/copy (IEEE binary32, no contraction);
<= 2 ulp from the oracle's SLEEF u10 results for sin/cos/tanh/log/exp/pow and
bit-exact for sqrt/abs.  Everything goes through the C ABI.
"""
import ctypes as C
import os

import numpy as np
import pytest

from helpers import assert_bit_equal, oracle_views, ulp_distance

pytestmark = pytest.mark.gpu

BINARY = ["add", "sub", "mul", "div"]


def dptr(t, offset=0):
    return C.c_void_p(t.ptr + 4 * offset)


@pytest.mark.parametrize("op", BINARY)
def test_binary_1d_stride_regimes(gpu, O, op):
    """waffe2_s<op>(n, x, incx, y, incy) for every (incx, incy) regime of
    cl-waffe2-simd.c:153-213 with incx >= 1, including n % 8 tails."""
    W = gpu
    rng = np.random.default_rng(11)
    fn = getattr(W.lib.get(), "wf2hip_s" + op)
    for n in [0, 1, 7, 8, 9, 255, 1000, 4099, 70001]:
        for incx, incy in [(1, 1), (1, 0), (2, 1), (1, 3), (2, 2), (3, 0)]:
            size = max(1, n) * 3 + 8
            x = rng.standard_normal(size).astype(np.float32)
            y = rng.standard_normal(size).astype(np.float32)
            want = x.copy()
            O.binary_1d(op, n, want, incx, y, incy)
            dx, dy = W.HIPTensor.from_numpy(x), W.HIPTensor.from_numpy(y)
            W.lib.check(fn(n, dptr(dx), incx, dptr(dy), incy))
            assert_bit_equal(dx.numpy(), want, f"{op} n={n} incx={incx} incy={incy}")


def test_binary_1d_unaligned_pointers(gpu, O):
    """Offsets that break 16-byte alignment must take the scalar path."""
    W = gpu
    rng = np.random.default_rng(12)
    for offx, offy in [(1, 0), (0, 3), (2, 1), (3, 3)]:
        x = rng.standard_normal(5000).astype(np.float32)
        y = rng.standard_normal(5000).astype(np.float32)
        want = x.copy()
        O.binary_1d("add", 4000, want, 1, y, 1, offx=offx, offy=offy)
        dx, dy = W.HIPTensor.from_numpy(x), W.HIPTensor.from_numpy(y)
        W.lib.check(W.lib.get().wf2hip_sadd(4000, dptr(dx, offx), 1, dptr(dy, offy), 1))
        assert_bit_equal(dx.numpy(), want, f"offsets {offx},{offy}")


def test_ieee_special_values(gpu):
    """Division and multiplication on denormals, signed zeros, infinities:
    correctly rounded, denormals preserved (closed form: numpy IEEE binary32)."""
    W = gpu
    tiny = np.float32(1e-45)
    vals = np.array([0.0, -0.0, 1.0, -1.0, tiny, -tiny, 1.1754944e-38, 3.4028235e38, np.inf,
                     -np.inf, 1e-40, 3.0, 7.0, 1e20, 1e-20, 0.1], np.float32)
    x = np.repeat(vals, len(vals))
    y = np.tile(vals, len(vals))
    for op, f in [("add", np.add), ("sub", np.subtract), ("mul", np.multiply), ("div", np.divide)]:
        with np.errstate(all="ignore"):
            want = f(x, y)
        dx, dy = W.HIPTensor.from_numpy(x), W.HIPTensor.from_numpy(y)
        W.lib.check(getattr(W.lib.get(), "wf2hip_s" + op)(x.size, dptr(dx), 1, dptr(dy), 1))
        assert_bit_equal(dx.numpy(), want, op)


def test_config1_contiguous(gpu, O):
    """benchmark configuration 1: Z1 = A + B, Z2 = A * B on (1024, 1024) N(0,1), seed 1,
    through !add / !mul (copy + in-place node)."""
    W = gpu
    F = W.functional
    rng = np.random.Generator(np.random.PCG64(1))
    A = rng.standard_normal((1024, 1024)).astype(np.float32)
    B = rng.standard_normal((1024, 1024)).astype(np.float32)
    dA, dB = F.from_numpy(A), F.from_numpy(B)
    for fn, op in [(F.add, "add"), (F.mul, "mul")]:
        want = A.copy().ravel()
        O.binary_1d(op, want.size, want, 1, B.ravel(), 1)
        assert_bit_equal(fn(dA, dB).numpy().ravel(), want, op)
    assert_bit_equal(dA.numpy(), A, "operands untouched")


def test_config2_views(gpu, O):
    """benchmark configuration 2: row-broadcast add, column-stride-2 slice times 0.5,
    subtraction of offset views -- against the oracle running the reference's
    own per-row schedule."""
    W = gpu
    F = W.functional
    rng = np.random.Generator(np.random.PCG64(2))
    A = rng.standard_normal((4096, 8192)).astype(np.float32)
    B = rng.standard_normal((1, 8192)).astype(np.float32)
    dA, dB = F.from_numpy(A), F.from_numpy(B)

    # A + B (B broadcast along rows): in place on a copy of A
    x = F.copy(dA)
    yb = dB.view((":broadcast", 4096), True)
    F.add_(x, yb)
    want = A.copy().ravel()
    v = oracle_views(O, [x, yb])
    cnt, _ = O.schedule(v, cap=1)
    assert cnt == 4096  # one sadd per row on the CPU
    O.node_nd("add", v, want, B.ravel().copy())
    assert_bit_equal(x.numpy().ravel(), want, "A + B broadcast")

    # A[:, 0:8192:2] * 0.5
    sl = dA.view(True, (0, 8192, 2))
    got = F.mul(sl, 0.5)
    assert got.shape == [4096, 4096]
    assert_bit_equal(got.numpy(), A[:, ::2] * np.float32(0.5), "strided slice * 0.5")

    # C = A[1024:3072, :] - A[0:2048, :]
    top, bot = dA.view((1024, 3072), True), dA.view((0, 2048), True)
    got = F.sub(top, bot)
    assert_bit_equal(got.numpy(), A[1024:3072] - A[0:2048], "offset views")


def test_disjoint_windows_of_one_buffer(gpu):
    """x[:, :h] += x[:, h:] -- two windows of one storage whose address ranges
    interleave but never share an element -- is an ordinary in-place op; windows
    that do share elements are refused (the CPU result would depend on loop order)."""
    W = gpu
    F = W.functional
    rng = np.random.default_rng(81)
    for rows, cols in [(64, 512), (33, 1030), (7, 10)]:
        h = cols // 2
        A = rng.standard_normal((rows, cols)).astype(np.float32)
        t = F.from_numpy(A)
        F.add_(t.view(True, (0, h)), t.view(True, (h, 2 * h)))
        want = A.copy()
        want[:, :h] += A[:, h:2 * h]
        assert_bit_equal(t.numpy(), want, f"x[:, :h] += x[:, h:], {rows}x{cols}")
        t = F.from_numpy(A)
        F.mul_(t.view((0, rows // 2), True), t.view((rows - rows // 2, rows), True))  # upper rows *= lower rows
        want = A.copy()
        want[:rows // 2] *= A[rows - rows // 2:]
        assert_bit_equal(t.numpy(), want, "rows against later rows")
        t = F.from_numpy(A)
        with pytest.raises(W.HIPError):
            F.add_(t.view(True, (0, h)), t.view(True, (1, h + 1)))
        with pytest.raises(W.HIPError):
            F.add_(t.view((0, rows - 1), True), t.view((1, rows), True))


def test_every_second_element_as_source(gpu):
    """A [::2] slice read into contiguous rows -- the copy behind every out-of-place
    op on such a view (two aligned 16-byte loads per four elements when the rows
    start 0 or 1 floats past a 16-byte boundary, the generic kernel otherwise):
    copies, in-place ops with the slice on the right, unary math; row lengths that
    are and are not multiples of four.  Closed form: numpy in binary32."""
    W = gpu
    F = W.functional
    rng = np.random.default_rng(79)
    f32 = np.float32
    for rows, pitch, start, count in [(9, 1000, 0, 500), (7, 1004, 1, 450), (5, 4100, 0, 2049), (3, 4100, 1, 131),
                                      (4, 1000, 2, 256), (6, 1001, 0, 400), (1, 70004, 1, 35001), (2, 2048, 3, 1000)]:
        base = rng.standard_normal((rows, pitch)).astype(f32)
        want_slice = base[:, start:start + 2 * count:2]
        t = F.from_numpy(base)
        v = t.view(True, (start, start + 2 * count, 2))
        assert v.shape == [rows, count]
        assert_bit_equal(F.copy(v).numpy(), want_slice, f"copy of [::2], rows {rows} pitch {pitch} start {start}")
        acc = rng.standard_normal((rows, count)).astype(f32)
        got = F.sub_(F.from_numpy(acc), v)
        assert_bit_equal(got.numpy(), acc - want_slice, f"x -= [::2], rows {rows} pitch {pitch} start {start}")
        got = F.mul(v, 0.5)  # the configured case: a copy of the slice, then the scalar product in place
        assert_bit_equal(got.numpy(), want_slice * f32(0.5), "0.5 * [::2]")
        got = F.abs(v)
        assert_bit_equal(got.numpy(), np.abs(want_slice), "abs of [::2]")
        assert_bit_equal(t.numpy(), base, "the source is untouched")
    # a 3-D source: slices of every matrix of a batch
    base = rng.standard_normal((3, 6, 520)).astype(f32)
    v = F.from_numpy(base).view(True, (1, 5), (0, 520, 2))
    assert_bit_equal(F.copy(v).numpy(), base[:, 1:5, 0:520:2], "3-D [::2] source")


def test_inplace_on_every_second_element(gpu):
    """In-place ops on [::2] slices (the kernel that stores whole vectors and
    writes the in-between elements back as read): row pitches and start columns
    that break the 16-byte alignment of the rows, every kind of second operand,
    the whole storage compared so that untouched elements are checked too; and
    the layout where rows interleave (an (n, 2) tensor seen as (2, n)), which must
    not take that kernel.  Closed form: IEEE binary32 arithmetic in numpy."""
    W = gpu
    F = W.functional
    rng = np.random.default_rng(77)
    f32 = np.float32
    for rows, pitch, start, count in [(5, 1000, 0, 500), (7, 1001, 1, 450), (3, 4099, 3, 2000),
                                      (4, 514, 2, 256), (1, 70001, 5, 30000), (6, 300, 0, 150)]:
        base = rng.standard_normal((rows, pitch)).astype(f32)
        sel = np.s_[:, start:start + 2 * count:2]
        for kind in ("scalar", "contiguous", "slice", "row", "column"):
            t = F.from_numpy(base)
            v = t.view(True, (start, start + 2 * count, 2))
            assert v.shape == [rows, count]
            want = base.copy()
            if kind == "scalar":
                F.mul_(v, 0.37)
                want[sel] *= f32(0.37)
            elif kind == "contiguous":
                y = rng.standard_normal((rows, count)).astype(f32)
                F.add_(v, F.from_numpy(y))
                want[sel] += y
            elif kind == "slice":
                ybase = rng.standard_normal((rows, 2 * count + 3)).astype(f32)
                F.sub_(v, F.from_numpy(ybase).view(True, (1, 1 + 2 * count, 2)))
                want[sel] -= ybase[:, 1:1 + 2 * count:2]
            elif kind == "row":
                y = (rng.standard_normal((1, count)) + 3.0).astype(f32)
                F.div_(v, F.from_numpy(y).view((":broadcast", rows), True))
                want[sel] /= y
            else:
                y = rng.standard_normal((rows, 1)).astype(f32)
                F.mul_(v, F.from_numpy(y).view(True, (":broadcast", count)))
                want[sel] *= y
            assert_bit_equal(t.numpy(), want, f"[::2] in place, {kind}, rows {rows} pitch {pitch} start {start}")
    # even and odd elements of one storage against each other
    base = rng.standard_normal((8, 2048)).astype(f32)
    t = F.from_numpy(base)
    F.add_(t.view(True, (0, 2046, 2)), t.view(True, (1, 2048, 2)))  # 1023 elements each (floor((to-from)/step))
    want = base.copy()
    want[:, 0:2046:2] += base[:, 1:2047:2]
    assert_bit_equal(t.numpy(), want, "even += odd")
    # interleaved rows
    base = rng.standard_normal((3000, 2)).astype(f32)
    y = rng.standard_normal((2, 3000)).astype(f32)
    t = F.from_numpy(base)
    F.add_(t.permute(1, 0), F.from_numpy(y))
    assert_bit_equal(t.numpy(), base + y.T, "(n, 2) seen as (2, n)")


def test_large_transposed_operands(gpu):
    """Operands whose unit-stride axes differ, large enough for the 128 x 128
    LDS tiles: copies, an in-place binary op with a transposed second operand
    and a unary op reading a transposed source, with ragged tile edges and outer
    (batch) axes.  Closed form: numpy on the same views; bit-exact (exp <= 2 ulp
    of float64)."""
    W = gpu
    F = W.functional
    rng = np.random.default_rng(128)
    # the last three have a multiple of 8 tiles along the destination's contiguous axis, where
    # the tiles are handed out in bands (128 x 128 tiles twice, 64 x 64 tiles once)
    for shape, order in [((2052, 2060), (1, 0)), ((3, 1100, 1284), (0, 2, 1)), ((2, 3, 1028, 1032), (0, 1, 3, 2)),
                         ((1284, 5, 1100), (2, 1, 0)), ((2048, 2100), (1, 0)), ((2, 2040, 1100), (0, 2, 1)),
                         ((3, 1020, 1100), (0, 2, 1))]:
        x = rng.standard_normal(shape).astype(np.float32)
        xt = np.transpose(x, order)
        dx = F.from_numpy(x)
        got = F.copy(dx.permute(*order))
        assert got.shape == list(xt.shape)
        assert_bit_equal(got.numpy(), np.ascontiguousarray(xt), f"copy {shape} -> {order}")
        y = rng.standard_normal(xt.shape).astype(np.float32)
        dy = F.from_numpy(y)
        F.sub_(dy, dx.permute(*order))
        assert_bit_equal(dy.numpy(), y - xt, f"sub_ {shape} -> {order}")
        e = F.exp(dx.permute(*order))
        assert ulp_distance(e.numpy(), np.exp(xt.astype(np.float64)).astype(np.float32)).max() <= 1


def _random_view(rng, n):
    """A random subscript for an axis of extent n."""
    k = rng.integers(0, 6)
    if k == 0 or n < 3:
        return True
    if k == 1:
        a = int(rng.integers(0, n - 1))
        b = int(rng.integers(a + 1, n + 1))
        return (a, b)
    if k == 2:
        a = int(rng.integers(0, n - 2))
        b = int(rng.integers(a + 2, n + 1))
        return (a, b, int(rng.integers(2, 4)))
    if k == 3:
        a = int(rng.integers(0, n - 2))
        b = int(rng.integers(a + 2, n + 1))
        return (a, b, -int(rng.integers(1, 3)))
    if k == 4:
        return int(rng.integers(0, n))
    return True


@pytest.mark.parametrize("seed", range(6))
def test_random_nd_views_match_reference_schedule(gpu, O, seed):
    """Random ranks/shapes/slices/broadcasts: the single N-D launch must equal
    the oracle executing the reference's host-loop schedule, bit for bit.
    Accumulation into broadcast destinations uses the sequential reduce mode."""
    W = gpu
    rng = np.random.default_rng(100 + seed)
    lib = W.lib.get()
    W.lib.check(lib.wf2hip_set_reduce_mode(1))
    try:
        for case in range(40):
            rank = int(rng.integers(1, 5))
            storage_shape = [int(rng.integers(1, 9)) if rng.random() < 0.7 else int(rng.integers(9, 40))
                             for _ in range(rank)]
            xs = rng.standard_normal(storage_shape).astype(np.float32)
            tx = W.HIPTensor.from_numpy(xs)
            vx = tx.view(*[_random_view(rng, n) for n in storage_shape])
            vis = vx.shape
            # y: its own storage whose visible shape equals x's, with broadcast axes
            y_storage, y_subs = [], []
            for n in vis:
                if n > 1 and rng.random() < 0.3:
                    y_storage.append(1)
                    y_subs.append((":broadcast", n))
                else:
                    pad = int(rng.integers(0, 3))
                    y_storage.append(n + pad)
                    y_subs.append((pad, n + pad) if pad else True)
            ys = (rng.standard_normal(y_storage) + 2.0).astype(np.float32)
            ty = W.HIPTensor.from_numpy(ys)
            vy = ty.view(*y_subs)
            assert vy.shape == vis
            op = ["add", "sub", "mul", "div", "move"][int(rng.integers(0, 5))]
            want = xs.copy().ravel()
            O.node_nd(op, oracle_views(O, [vx, vy]), want, ys.ravel().copy())
            W.forward({"add": "AddNode", "sub": "SubNode", "mul": "MulNode", "div": "DivNode",
                       "move": "MoveTensorNode"}[op], vx, vy)
            assert_bit_equal(tx.storage_numpy(), want,
                             f"case {case} op {op} x{storage_shape}{[v.view for v in vx.views]} "
                             f"y{y_storage}{y_subs}")
    finally:
        W.lib.check(lib.wf2hip_set_reduce_mode(0))


@pytest.mark.parametrize("op", BINARY + ["move"])
def test_broadcast_destination_sequential_mode(gpu, O, op):
    """x viewed (:broadcast n): x[0] <- x[0] op y[i] in storage order, the
    reference's incx == 0 loop (cl-waffe2-simd.c:205-212)."""
    W = gpu
    rng = np.random.default_rng(21)
    lib = W.lib.get()
    W.lib.check(lib.wf2hip_set_reduce_mode(1))
    try:
        for shape, bc in [((6, 50), (False, True)), ((6, 50), (True, False)), ((4, 5, 33), (True, False, True)),
                          ((300,), (True,)), ((3, 4, 5), (True, True, True))]:
            xshape = [1 if b else n for n, b in zip(shape, bc)]
            xs = rng.uniform(0.5, 1.5, xshape).astype(np.float32)
            ys = rng.uniform(0.9, 1.1, shape).astype(np.float32)
            tx, ty = W.HIPTensor.from_numpy(xs), W.HIPTensor.from_numpy(ys)
            vx = tx.view(*[(":broadcast", n) if b else True for n, b in zip(shape, bc)])
            want = xs.copy().ravel()
            O.node_nd(op, oracle_views(O, [vx, ty]), want, ys.ravel().copy())
            W.forward({"add": "AddNode", "sub": "SubNode", "mul": "MulNode", "div": "DivNode",
                       "move": "MoveTensorNode"}[op], vx, ty)
            assert_bit_equal(tx.storage_numpy(), want, f"{op} {shape} {bc}")
    finally:
        W.lib.check(lib.wf2hip_set_reduce_mode(0))


def test_copy_layouts(gpu):
    """MoveTensorNode on transposed / permuted / strided sources (the tile and
    generic kernels), against numpy indexing; includes the reference docstring
    vector ->contiguous(!t (ax+b (3 3) 1 0)) = #(0 3 6 1 4 7 2 5 8)
    (base-impl/fundamental.lisp:1070-1097)."""
    W = gpu
    F = W.functional
    a = np.arange(9, dtype=np.float32).reshape(3, 3)
    got = F.copy(F.from_numpy(a).permute(1, 0))
    assert got.storage_numpy().tolist() == [0, 3, 6, 1, 4, 7, 2, 5, 8]
    rng = np.random.default_rng(5)
    for shape, order in [((257, 130), (1, 0)), ((3, 70, 65), (0, 2, 1)), ((2, 33, 12, 64), (0, 2, 1, 3)),
                         ((5, 6, 7), (2, 1, 0)), ((64, 64), (1, 0)), ((2, 3, 100, 40), (3, 1, 0, 2))]:
        x = rng.standard_normal(shape).astype(np.float32)
        got = F.copy(F.from_numpy(x).permute(*order))
        assert_bit_equal(got.numpy(), np.transpose(x, order), f"permute {shape} {order}")
    x = rng.standard_normal((40, 100)).astype(np.float32)
    rows = W.make_range(3, 37, 2).indices()
    cols = W.make_range(0, 99, -3).indices()  # walks down from 96
    assert cols[0] == 96 and cols[-1] == 0
    got = F.copy(F.from_numpy(x).view((3, 37, 2), (0, 99, -3)))
    assert_bit_equal(got.numpy(), x[np.ix_(rows, cols)], "stepped and reversed slices")


def test_overlap_is_rejected(gpu):
    W = gpu
    a = W.HIPTensor.from_numpy(np.arange(100, dtype=np.float32))
    with pytest.raises(W.HIPError) as e:
        W.forward("SubNode", a.view((10, 60)), a.view((0, 50)))
    assert e.value.code == W.lib.EOVERLAP
    # the same window on both sides is fine: x <- x + x
    W.forward("AddNode", a.view((10, 60)), a.view((10, 60)))
    want = np.arange(100, dtype=np.float32)
    want[10:60] *= 2
    assert_bit_equal(a.numpy(), want)


def test_invalid_arguments(gpu):
    W = gpu
    lib = W.lib.get()
    v = W.lib.View2()
    v.rank = 9
    assert lib.wf2hip_binary_nd(0, C.byref(v), None, None) == -1
    assert b"rank" in lib.wf2hip_last_error()
    assert lib.wf2hip_sadd(-1, None, 1, None, 1) == -1
    assert lib.wf2hip_sadd(4, None, 1, None, 1) == -1
    assert lib.wf2hip_sadd(0, None, 1, None, 1) == 0  # empty: nothing to do
    with pytest.raises(ValueError):
        W.forward("AddNode", W.HIPTensor([2, 3]), W.HIPTensor([3, 2]))


# ---------------------------------------------------------------------------
# unary
# ---------------------------------------------------------------------------

CFG3 = [("exp", -10, 10), ("tanh", -10, 10), ("sin", -100, 100), ("log", 1e-3, 1e3),
        ("cos", -100, 100)]


@pytest.mark.parametrize("op,lo,hi", CFG3)
def test_config3_transcendentals(gpu, O, op, lo, hi):
    """benchmark configuration 3 ranges (seed 3) on 2^22 elements: <= 2 ulp from the
    oracle's SLEEF u10 results and <= 1 ulp from float64 truth."""
    W = gpu
    rng = np.random.Generator(np.random.PCG64(3))
    n = 1 << 22
    x = rng.uniform(lo, hi, n).astype(np.float32)
    want = np.zeros(n, np.float32)
    O.unary_1d(op, n, x, 1, want, 1)
    dx = W.HIPTensor.from_numpy(x)
    out = W.HIPTensor([n])
    W.lib.check(getattr(W.lib.get(), "wf2hip_s" + op)(n, dptr(dx), 1, dptr(out), 1))
    got = out.numpy()
    assert O.sleef_available(), "oracle fell back to libm: SLEEF provider missing"
    assert ulp_distance(got, want).max() <= 2
    truth = getattr(np, op)(x.astype(np.float64)).astype(np.float32)
    assert ulp_distance(got, truth).max() <= 1


@pytest.mark.parametrize("op,lo,hi", CFG3[:4])
def test_config3_full_size(gpu, O, op, lo, hi):
    """benchmark configuration 3 at its full size, 2^26 elements in one flat call (the
    non-temporal streaming kernel): same bars as above."""
    W = gpu
    rng = np.random.Generator(np.random.PCG64(3))
    n = 1 << 26
    x = rng.uniform(lo, hi, n).astype(np.float32)
    want = np.zeros(n, np.float32)
    O.unary_1d(op, n, x, 1, want, 1)
    dx = W.HIPTensor.from_numpy(x)
    out = W.HIPTensor([n])
    W.lib.check(getattr(W.lib.get(), "wf2hip_s" + op)(n, dptr(dx), 1, dptr(out), 1))
    got = out.numpy()
    del dx, out
    assert ulp_distance(got, want).max() <= 2
    truth = getattr(np, op)(x.astype(np.float64)).astype(np.float32)
    assert ulp_distance(got, truth).max() <= 1


def test_metric_size_binary_and_rowsum(gpu, O):
    """The benchmark's workload, (8192, 8192) = 2^26 elements from seed 6:
    x += y and x *= y bit-exact against the oracle, row sums <= 1e-5 relative
    to the float64 sums (relative to sum |x|, the forward error scale)."""
    W = gpu
    F = W.functional
    rng = np.random.Generator(np.random.PCG64(6))
    X = rng.standard_normal((8192, 8192)).astype(np.float32)
    Y = rng.standard_normal((8192, 8192)).astype(np.float32)
    dX, dY = F.from_numpy(X), F.from_numpy(Y)
    for op in ("add", "mul"):
        want = X.copy().ravel()
        O.binary_1d(op, want.size, want, 1, Y.ravel(), 1)
        work = F.copy(dX)
        getattr(F, op + "_")(work, dY)
        assert_bit_equal(work.numpy().ravel(), want, op)
        del work, want
    got = F.sum(dY, axis=1).numpy().ravel().astype(np.float64)
    truth = Y.astype(np.float64).sum(axis=1)
    scale = np.abs(Y).astype(np.float64).sum(axis=1)
    assert np.max(np.abs(got - truth) / scale) <= 1e-5
    # one rounding of the float64 sum is the best any fp32 result can do
    assert np.max(np.abs(got - truth) / np.maximum(np.abs(truth), 1e-30) * (np.abs(truth) > 1)) <= 1e-6


MORE_UNARY = [("tan", -100, 100), ("asin", -1, 1), ("acos", -1, 1), ("atan", -100, 100), ("sinh", -10, 10),
              ("cosh", -10, 10), ("log2", 1e-3, 1e3), ("log10", 1e-3, 1e3), ("log1p", -0.99, 100)]
MORE_TRUTH = {"tan": np.tan, "asin": np.arcsin, "acos": np.arccos, "atan": np.arctan, "sinh": np.sinh,
              "cosh": np.cosh, "log2": np.log2, "log10": np.log10, "log1p": np.log1p}


@pytest.mark.parametrize("op,lo,hi", MORE_UNARY)
def test_more_unary_functions(gpu, O, op, lo, hi):
    """Tan, ASin, ACos, ATan, SinH, CosH, Log2, Log10, Log1p through the nodes
    on 2^22 elements: <= 2 ulp from the oracle's SLEEF u10 results, <= 1 ulp
    from float64; then the reference's golden special values, strides and an
    n % 8 tail through the 1-D entry points."""
    W = gpu
    F = W.functional
    rng = np.random.Generator(np.random.PCG64(33))
    n = 1 << 22
    x = rng.uniform(lo, hi, n).astype(np.float32)
    want = np.zeros(n, np.float32)
    O.unary_1d(op, n, x, 1, want, 1)
    got = getattr(F, op)(F.from_numpy(x)).numpy()
    assert O.sleef_available()
    assert ulp_distance(got, want).max() <= 2
    assert ulp_distance(got, MORE_TRUTH[op](x.astype(np.float64)).astype(np.float32)).max() <= 1
    gold = np.load(os.path.join(os.path.dirname(__file__), "golden", "unary_more_kernels.npz"))
    edge = gold["edge_x"]
    lib = W.lib.get()
    dx, dout = W.HIPTensor.from_numpy(edge), W.HIPTensor([edge.size])
    W.lib.check(getattr(lib, "wf2hip_s" + op)(edge.size, dptr(dx), 1, dptr(dout), 1))
    ref = gold[f"un_{op}_edge_out"].copy()
    with np.errstate(all="ignore"):
        truth = MORE_TRUTH[op](edge.astype(np.float64)).astype(np.float32)
    early = np.isinf(ref) & np.isfinite(truth)      # SLEEF's sinhf / coshf overflow early (88.72 .. 89.42)
    ref[early] = truth[early]
    assert ulp_distance(dout.numpy(), ref).max() <= 2
    xs = gold[f"un_{op}_range_x"]
    dxs = W.HIPTensor.from_numpy(xs)
    for cnt, incx, inco in [(13, 2, 1), (16, 1, 3), (9, 0, 1)]:
        dst = W.HIPTensor.from_numpy(np.full(64, 7.0, np.float32))
        W.lib.check(getattr(lib, "wf2hip_s" + op)(cnt, dptr(dxs), incx, dptr(dst), inco))
        assert ulp_distance(dst.numpy(), gold[f"un_{op}_{cnt}_{incx}_{inco}_out"]).max() <= 2


def test_inv(gpu, O):
    """wf2hip_sinv against the oracle, bit for bit, strided and stride 0."""
    W = gpu
    lib = W.lib.get()
    rng = np.random.default_rng(6)
    x = np.concatenate([rng.standard_normal(5000), [0.0, -0.0, np.inf, 1e-45, 3e38, 1.0, 3.0]]).astype(np.float32)
    for n, inc in [(x.size, 1), (x.size // 2, 2), (100, 7), (6, 0), (0, 1)]:
        want = x.copy()
        with np.errstate(all="ignore"):
            O.inv_1d(n, want, inc)
        dx = W.HIPTensor.from_numpy(x)
        W.lib.check(lib.wf2hip_sinv(n, dptr(dx), inc))
        assert_bit_equal(dx.numpy(), want, f"inv n={n} inc={inc}")


def test_unary_edge_values_and_tails(gpu, O):
    """+-0, denormals, +-inf, NaN, huge arguments, n % 8 != 0 tails, strided
    in/out."""
    W = gpu
    lib = W.lib.get()
    edge = np.array([0.0, -0.0, 1e-45, -1e-45, 1e-39, 1.0, -1.0, np.inf, -np.inf, np.nan, 88.72, 88.73,
                     -87.4, -103.9, -104.5, 1e10, -1e10, 3.4e38, 1e6, 1.5e6, 9.01, -9.01, 0.5, 2.0,
                     1e-3, 123456.7, 1e-20, 0.99999994, 1.0000001, 3.1415927, 1.5707964, 6.2831855,
                     102.1, 355.0, 710.0, 1e5, 65536.0], np.float32)
    for op in ["exp", "tanh", "sin", "cos", "log", "sqrt", "abs"]:
        for n, incx, inco in [(edge.size, 1, 1), (edge.size, 1, 2), (13, 2, 1), (5, 3, 3)]:
            want = np.full(edge.size * 3, 7.0, np.float32)
            with np.errstate(all="ignore"):
                O.unary_1d(op, n, edge, incx, want, inco)
            dx = W.HIPTensor.from_numpy(edge)
            out = W.HIPTensor.from_numpy(np.full(edge.size * 3, 7.0, np.float32))
            W.lib.check(getattr(lib, "wf2hip_s" + op)(n, dptr(dx), incx, dptr(out), inco))
            got = out.numpy()
            limit = 0 if op in ("sqrt", "abs") else 2
            d = ulp_distance(got, want)
            assert d.max() <= limit, (op, n, incx, inco, edge[np.argmax(d[::inco][:n])] if inco else None,
                                      got[np.argmax(d)], want[np.argmax(d)])


def test_unary_source_broadcast(gpu, O):
    """incx == 0: the reference takes the libm-in-double scalar path for the
    whole range (cl-waffe2-simd.c:592,636-641)."""
    W = gpu
    x = np.array([1.2345], np.float32)
    want = np.zeros(37, np.float32)
    O.unary_1d("exp", 37, x, 0, want, 1)
    out = W.HIPTensor([37])
    W.lib.check(W.lib.get().wf2hip_sexp(37, dptr(W.HIPTensor.from_numpy(x)), 0, dptr(out), 1))
    assert ulp_distance(out.numpy(), want).max() <= 2


@pytest.mark.parametrize("p", [2.0, 3.0, 0.5, 2.5, -1.0, 0.0, 1.0, -2.0, 7.0])
def test_pow(gpu, O, p):
    """ExptNode: x^p, <= 2 ulp from SLEEF powf u10 (GELU uses p = 3, LayerNorm
    p = 2)."""
    W = gpu
    rng = np.random.default_rng(8)
    n = 100003
    x = rng.uniform(0.01, 30.0, n).astype(np.float32)
    if p == int(p):
        x[::2] *= -1  # integral exponents are defined for negative bases
    want = np.zeros(n, np.float32)
    O.pow_1d(n, x, 1, p, want, 1)
    out = W.functional.expt(W.HIPTensor.from_numpy(x), p)
    assert ulp_distance(out.numpy(), want).max() <= 2


def test_gelu_known_answer(gpu):
    """The reference's own exact-equality check: GELU(1.0) = 0.841192
    (vm/nodes/t/composite.lisp:119,132,146), through the node-for-node recipe
    and through the fused kernel."""
    W = gpu
    F = W.functional
    one = F.from_numpy(np.ones((2, 3), np.float32))
    for fn in (F.gelu, F.gelu_fused):
        got = fn(one).numpy()
        assert np.all(np.abs(got - 0.841192) < 5e-7), got
    x = np.random.default_rng(0).standard_normal((64, 100)).astype(np.float32) * 3
    truth = x.astype(np.float64)
    truth = truth / (1.0 + np.exp(-2.0 * 0.7978845608028654 * (truth + 0.044715 * truth ** 3)))
    assert ulp_distance(F.gelu_fused(F.from_numpy(x)).numpy(), truth.astype(np.float32)).max() <= 2
    np.testing.assert_allclose(F.gelu(F.from_numpy(x)).numpy(), truth, rtol=2e-5, atol=2e-6)


LISP_LOOP_NODES = [("sign", -3, 3), ("square", -100, 100), ("asinh", -1e4, 1e4), ("acosh", 1, 1e4),
                   ("atanh", -0.999, 0.999)]


@pytest.mark.parametrize("op,lo,hi", LISP_LOOP_NODES)
def test_nodes_the_cpu_backend_leaves_to_lisptensor(gpu, O, op, lo, hi):
    """SignNode, SquareNode, ASinHNode, ACosHNode, ATanHNode (the CPU backend has no impl;
    LispTensor's loop would be handed a device handle): against the oracle's restatement
    of that loop and against float64 on 2^20 elements -- sign and square bit-exact, the
    inverse hyperbolic functions within 1 ulp -- on a strided view, on :double, and on
    the special values."""
    W = gpu
    F = W.functional
    rng = np.random.Generator(np.random.PCG64(34))
    n = 1 << 20
    x = rng.uniform(lo, hi, n).astype(np.float32)
    want = np.zeros(n, np.float32)
    O.unary_1d(op, n, x, 1, want, 1)
    got = getattr(F, op)(F.from_numpy(x)).numpy()
    limit = 0 if op in ("sign", "square") else 1
    assert ulp_distance(got, want).max() <= limit
    # CL's signum keeps the sign of a zero, numpy's sign does not
    truth = {"sign": lambda v: np.where(v == 0, v, np.sign(v)), "square": np.square, "asinh": np.arcsinh,
             "acosh": np.arccosh, "atanh": np.arctanh}[op]
    assert ulp_distance(got, truth(x.astype(np.float64)).astype(np.float32)).max() <= limit
    # a strided, offset view as source and a column of a matrix as destination
    src = F.from_numpy(x[:6000].reshape(60, 100)).view((5, 55), (3, 99, 2))
    dst = W.HIPTensor([50, 48])
    getattr(F, op)(src, out=dst)
    assert ulp_distance(dst.numpy(), truth(x[:6000].reshape(60, 100)[5:55, 3:99:2].astype(np.float64))
                        .astype(np.float32)).max() <= limit
    # :double tensors go through the binary64 routines
    xd = x[:5000].astype(np.float64)
    gotd = getattr(F, op)(F.from_numpy(xd, dtype="double")).numpy()
    np.testing.assert_allclose(gotd, truth(xd), rtol=4e-16, atol=0)
    edge = np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 1.0, -1.0, 0.5, 1e-30, -1e-30, 3e38], np.float32)
    with np.errstate(all="ignore"):
        te = truth(edge.astype(np.float64)).astype(np.float32)
    ge = getattr(F, op)(F.from_numpy(edge)).numpy()
    assert ulp_distance(ge, te).max() <= limit, (edge, ge, te)
    assert np.array_equal(np.signbit(ge[~np.isnan(te)]), np.signbit(te[~np.isnan(te)]))


@pytest.mark.parametrize("seed", range(40))
def test_random_permuted_and_sliced_passes(gpu, seed):
    """Random ranks, extents (short, odd, just past a tile), axis orders and windows: copies out of and into
    permuted views, an accumulating pass into a permuted destination and a unary pass over one, against
    numpy's indexing.  Data movement and single roundings: bit-exact.  Whatever kernel the dispatcher picks
    for the layout (rows, tiles, narrow tiles, strided gathers, an element per lane) must agree."""
    F = gpu.functional
    rng = np.random.default_rng(1000 + seed)
    extents = [1, 2, 3, 5, 8, 13, 16, 17, 31, 32, 33, 64, 100, 257, 300, 513]
    rank = int(rng.integers(2, 5))
    while True:
        shape = [int(rng.choice(extents)) for _ in range(rank)]
        if np.prod(shape) <= 300000:
            break
    perm = tuple(int(p) for p in rng.permutation(rank))
    x = rng.standard_normal(shape).astype(np.float32)
    dx = F.from_numpy(x)
    # a window on one axis (start past 0, so that the base pointer loses its alignment)
    axis = int(rng.integers(0, rank))
    lo = int(rng.integers(0, max(1, shape[axis] // 3) + 1)) if shape[axis] > 1 else 0
    hi = shape[axis] - int(rng.integers(0, 2)) if shape[axis] - lo > 1 else shape[axis]
    subs = [True] * rank
    subs[axis] = (lo, hi)
    index = tuple(slice(lo, hi) if a == axis else slice(None) for a in range(rank))
    xv, dv = x[index], dx.view(*subs)
    # copy out of a permuted window
    assert_bit_equal(F.copy(dv.permute(*perm)).numpy(), xv.transpose(perm), f"copy {shape} {perm} axis {axis} [{lo}:{hi}]")
    # unary pass over it
    assert_bit_equal(F.abs(dv.permute(*perm)).numpy(), np.abs(xv.transpose(perm)), "abs")
    # accumulate into the permuted window, then copy into it
    y = rng.standard_normal(xv.transpose(perm).shape).astype(np.float32)
    dy = F.from_numpy(y)
    want = x.copy()
    want[index] = xv + y.transpose(np.argsort(perm))
    F.add_(dv.permute(*perm), dy)
    assert_bit_equal(dx.numpy(), want, "accumulate into the permuted window")
    want[index] = y.transpose(np.argsort(perm))
    F.move_(dv.permute(*perm), dy)
    assert_bit_equal(dx.numpy(), want, "copy into the permuted window")
