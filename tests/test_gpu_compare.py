"""Where-Operation-Node / Compare-Operation-Node kernels against the oracle
(which is pinned bitwise to the reference's compiled waffe2_s{eq,lt,le,gt,ge}
[_scal] by tests/test_oracle_golden.py).  Results are one of two constants, so
the bar is bit equality everywhere."""
import ctypes as C

import numpy as np
import pytest

from helpers import assert_bit_equal, oracle_views

pytestmark = pytest.mark.gpu

OPS = ["eq", "lt", "le", "gt", "ge"]
SYMBOL = {"eq": "=", "lt": "<", "le": "<=", "gt": ">", "ge": ">="}
REGIMES = [(1, 1, 1), (1, 0, 1), (2, 1, 1), (1, 3, 2), (2, 2, 3), (0, 1, 1), (1, 1, 0), (3, 0, 0), (0, 0, 0)]


def dptr(t, off=0):
    return C.c_void_p(t.ptr + 4 * off)


@pytest.mark.parametrize("op", OPS)
def test_compare_1d_stride_regimes(gpu, O, op):
    W = gpu
    lib = W.lib.get()
    rng = np.random.default_rng(hash(op) % 1000)
    for n in (0, 1, 3, 4, 7, 8, 9, 31, 64, 67, 1000, 4099):
        for incx, incy, inco in REGIMES:
            size = max(n, 1) * 3 + 1
            x = rng.integers(-3, 4, size).astype(np.float32)
            y = rng.integers(-3, 4, size).astype(np.float32)
            x[rng.integers(0, size, 3)] = np.nan
            for scal in (False, True):
                want = np.full(size, 9.0, np.float32)
                dout = W.HIPTensor.from_numpy(want)
                dx, dy = W.HIPTensor.from_numpy(x), W.HIPTensor.from_numpy(y)
                if scal:
                    O.cmp_scal_1d(op, n, x, incx, want, inco, 1.0, 2.5, -1.5)
                    W.lib.check(getattr(lib, f"wf2hip_s{op}_scal")(n, dptr(dx), incx, dptr(dout), inco,
                                                                   1.0, 2.5, -1.5))
                else:
                    O.cmp_1d(op, n, x, incx, y, incy, want, inco, 2.5, -1.5)
                    W.lib.check(getattr(lib, f"wf2hip_s{op}")(n, dptr(dx), incx, dptr(dy), incy, dptr(dout),
                                                              inco, 2.5, -1.5))
                assert_bit_equal(dout.numpy(), want, f"{op} n={n} inc=({incx},{incy},{inco}) scal={scal}")


@pytest.mark.parametrize("op", OPS)
def test_compare_special_values(gpu, op):
    """Every special value against every other: NaN is false under all five
    predicates, -0 equals +0 (numpy's IEEE comparisons are the closed form)."""
    F = gpu.functional
    edge = np.array([0.0, -0.0, 1.0, -1.0, np.nan, np.inf, -np.inf, 1e-45, -1e-45, 3.4e38, 0.5, 2.0,
                     -2.0, 1.0000001, 0.99999994, 7.0], np.float32)
    xs, ys = np.repeat(edge, edge.size), np.tile(edge, edge.size)
    f = {"eq": np.equal, "lt": np.less, "le": np.less_equal, "gt": np.greater, "ge": np.greater_equal}[op]
    with np.errstate(invalid="ignore"):
        want = f(xs, ys).astype(np.float32)
    got = F.compare(F.from_numpy(xs), F.from_numpy(ys), SYMBOL[op]).numpy()
    assert_bit_equal(got, want, op)
    for s in edge:
        with np.errstate(invalid="ignore"):
            want = np.where(f(edge, s), np.float32(3.0), np.float32(-7.0))
        got = F.where(F.from_numpy(edge), SYMBOL[op], float(s), 3.0, -7.0).numpy()
        assert_bit_equal(got, want, f"{op} scal {s}")


def _random_view(rng, n):
    k = int(rng.integers(0, 5)) if n >= 3 else 0
    if k == 1:
        a = int(rng.integers(0, n - 1))
        return (a, int(rng.integers(a + 1, n + 1)))
    if k == 2:
        a = int(rng.integers(0, n - 2))
        return (a, int(rng.integers(a + 2, n + 1)), int(rng.integers(2, 4)))
    if k == 3:
        a = int(rng.integers(0, n - 2))
        return (a, int(rng.integers(a + 2, n + 1)), -int(rng.integers(1, 3)))
    return True


def _operand(W, rng, vis, allow_broadcast):
    """Fresh storage whose view has the visible shape `vis`: padded windows and,
    for inputs, (:broadcast n) axes."""
    storage, subs = [], []
    for n in vis:
        if allow_broadcast and n > 1 and rng.random() < 0.3:
            storage.append(1)
            subs.append((":broadcast", n))
        else:
            pad = int(rng.integers(0, 3))
            storage.append(n + pad)
            subs.append((pad, n + pad) if pad else True)
    host = rng.integers(-2, 3, storage).astype(np.float32)
    dev = W.HIPTensor.from_numpy(host)
    view = dev.view(*subs)
    assert list(view.shape) == list(vis)
    return host, dev, view


@pytest.mark.parametrize("seed", range(4))
def test_compare_nd_views_match_reference_schedule(gpu, O, seed):
    """Random sliced / strided / reversed / broadcast views of three tensors:
    the single launch equals the oracle executing the reference's loop schedule
    with one 1-D call per row (backends/cpu/logical.lisp:37-84)."""
    W = gpu
    F = W.functional
    rng = np.random.default_rng(900 + seed)
    for case in range(30):
        rank = int(rng.integers(1, 5))
        storage_shape = [int(rng.integers(1, 9)) if rng.random() < 0.7 else int(rng.integers(9, 40))
                         for _ in range(rank)]
        xs = rng.integers(-2, 3, storage_shape).astype(np.float32)
        tx = W.HIPTensor.from_numpy(xs)
        vx = tx.view(*[_random_view(rng, n) for n in storage_shape])
        vis = vx.shape
        ys, ty, vy = _operand(W, rng, vis, True)
        os_, to, vo = _operand(W, rng, vis, False)
        op = OPS[case % 5]
        want = os_.copy().ravel()
        O.compare_nd(op, oracle_views(O, [vx, vy, vo]), xs.ravel().copy(), ys.ravel().copy(), want, 4.0, -4.0)
        F.compare(vx, vy, SYMBOL[op], 4.0, -4.0, out=vo)
        assert_bit_equal(to.storage_numpy(), want, f"case {case} compare {op} {storage_shape}")
        want = os_.copy().ravel()
        O.where_nd(op, oracle_views(O, [vx, vo]), xs.ravel().copy(), want, 0.0, 1.0, 0.0)
        to2 = W.HIPTensor.from_numpy(os_)
        vo2 = to2.view(*[v.view for v in vo.views])
        F.where(vx, SYMBOL[op], 0.0, out=vo2)
        assert_bit_equal(to2.storage_numpy(), want, f"case {case} where {op} {storage_shape}")


def test_relu_and_sigmoid(gpu):
    """!relu = x * (x > 0) (source/nn/activation.lisp:26): max(x, 0) with -0 for
    negative inputs times 0... the product form keeps the sign of zero of x * 0;
    !sigmoid within 4 ulp of the float64 value (four rounded operations)."""
    F = gpu.functional
    rng = np.random.default_rng(3)
    x = rng.standard_normal((37, 129)).astype(np.float32) * 3
    x[0, :4] = [0.0, -0.0, np.inf, -np.inf]
    got = F.relu(F.from_numpy(x)).numpy()
    with np.errstate(invalid="ignore"):
        want = x * (x > 0).astype(np.float32)
    assert_bit_equal(got, want, "relu")
    finite = np.isfinite(x)
    assert np.array_equal(got[finite], np.maximum(x[finite], 0.0))
    s = F.sigmoid(F.from_numpy(x)).numpy()
    truth = 1.0 / (1.0 + np.exp(-x.astype(np.float64)))
    err = np.abs(s.astype(np.float64) - truth) / np.spacing(truth.astype(np.float32)).astype(np.float64)
    assert err[finite].max() <= 4


def test_compare_full_size(gpu):
    """2^26 elements through the streaming kernel; ReLU at the benchmark size via the
    identity relu(x) + relu(-x) = |x| (bitwise)."""
    F = gpu.functional
    rng = np.random.Generator(np.random.PCG64(8))
    x = rng.standard_normal(1 << 26).astype(np.float32)
    y = rng.standard_normal(1 << 26).astype(np.float32)
    dx, dy = F.from_numpy(x), F.from_numpy(y)
    got = F.compare(dx, dy, "<", 1.0, 0.0).numpy()
    assert np.array_equal(got, (x < y).astype(np.float32))
    del got
    pos = F.relu(dx)
    neg = F.relu(F.mul(dx, -1.0))
    assert_bit_equal(F.add(pos, neg).numpy(), np.abs(x), "relu identity")


def test_compare_argument_checks(gpu):
    W = gpu
    F = W.functional
    a = W.HIPTensor([8])
    with pytest.raises(W.nodes.NodeNotFound):
        F.where(a, "evenp", 0.0)
    with pytest.raises(ValueError):
        F.compare(a, W.HIPTensor([9]), "<")
    # out overlapping x with a different mapping is refused, identical mapping is in place
    buf = W.HIPTensor.from_numpy(np.arange(16, dtype=np.float32))
    lo, hi = buf.view((0, 8)), buf.view((4, 12))
    with pytest.raises(W.HIPError) as e:
        F.compare(lo, lo, "=", out=hi)
    assert e.value.code == W.lib.EOVERLAP
    F.compare(lo, lo, "=", out=lo)
    assert np.array_equal(buf.numpy()[:8], np.ones(8, np.float32))


# ---------------------------------------------------------------------------
# MaxValue / MinValue / ArgMax / ArgMin nodes
# ---------------------------------------------------------------------------

@pytest.mark.parametrize("shape", [(5, 7), (1, 1), (3, 1000), (300, 33), (4, 5, 6), (2, 3, 4, 50), (64, 4096),
                                   (2, 40000), (1, 300000)])
def test_select_rows(gpu, O, shape):
    """Row-wise max / min / argmax / argmin through the nodes: values bitwise
    equal to the oracle's waffe2_s{max,min} restatement per row, indices equal to
    the first occurrence (small integers make ties frequent)."""
    W = gpu
    F = W.functional
    rng = np.random.default_rng(sum(shape))
    x = rng.integers(-50, 51, shape).astype(np.float32)
    dx = F.from_numpy(x)
    rows = x.reshape(-1, shape[-1])
    want_max = np.array([O.maxmin_1d("max", r.size, np.ascontiguousarray(r), 1) for r in rows[:64]], np.float32)
    got = F.max(dx).numpy()
    kept = got.shape
    assert kept == (shape[0], 1)
    flat = x.reshape(shape[0], -1)  # the reference reduces everything behind the kept axes
    assert_bit_equal(got.ravel(), flat.max(axis=1), "max")
    assert_bit_equal(F.min(dx).numpy().ravel(), flat.min(axis=1), "min")
    if len(shape) == 2:
        assert_bit_equal(got.ravel()[:64], want_max, "max vs oracle")
    am = F.argmax(dx).numpy()
    assert am.dtype == np.uint32 and am.shape == (shape[0], 1)
    assert np.array_equal(am.ravel(), flat.argmax(axis=1))
    assert np.array_equal(F.argmin(dx).numpy().ravel(), flat.argmin(axis=1))
    for r in range(min(shape[0], 8)):
        row = np.ascontiguousarray(flat[r])
        assert am.ravel()[r] == O.argmaxmin_1d("max", row.size, row, 1)


def test_select_axis_views_and_keepdims(gpu, O):
    """axis semantics of the reference ((butlast shape axis) kept), strided and
    offset sources, keepdims broadcast view."""
    W = gpu
    F = W.functional
    rng = np.random.default_rng(5)
    x = rng.standard_normal((6, 5, 8)).astype(np.float32)
    dx = F.from_numpy(x)
    assert_bit_equal(F.max(dx, axis=1).numpy(), x.reshape(6, 5, 8).max(axis=2, keepdims=True), "axis=1 keeps two")
    assert_bit_equal(F.max(dx, axis=2).numpy(), x.reshape(6, 40).max(axis=1, keepdims=True), "axis=2 keeps one")
    k = F.max(dx, axis=1, keepdims=True)
    assert k.shape == [6, 5, 8]
    assert_bit_equal(k.numpy(), np.broadcast_to(x.max(axis=2, keepdims=True), x.shape), "keepdims")
    # a strided window as the source of the node itself (no reshape in between)
    big = rng.standard_normal((10, 64)).astype(np.float32)
    db = F.from_numpy(big)
    win = db.view((2, 9), (3, 60, 2))
    out = W.HIPTensor([7, 1])
    W.forward("MaxValue-Node", win, out)
    sub = win.numpy()   # 28 columns: the reference's range size is floor(|from - to| / step)
    assert sub.shape == (7, 28) and np.array_equal(sub, big[2:9, 3:59:2])
    assert_bit_equal(out.numpy().ravel(), sub.max(axis=1), "strided max")
    iout = W.HIPTensor([7, 1], dtype="uint32")
    W.forward("ArgMin-Node", win, iout)
    assert np.array_equal(iout.numpy().ravel(), sub.argmin(axis=1))
    for r in range(7):
        assert out.numpy().ravel()[r] == O.maxmin_1d("max", sub.shape[1], np.ascontiguousarray(big[2 + r, 3:]), 2)
    with pytest.raises(ValueError):
        W.forward("ArgMax-Node", win, out)          # indices need a :uint32 destination


def test_select_many_short_rows(gpu):
    """Rows of at most one vector per lane, four to a wavefront: max / min / argmax /
    argmin against numpy (first occurrence), ragged row counts and lengths."""
    W = gpu
    F = W.functional
    rng = np.random.default_rng(113)
    for rows, cols in [(40000, 10), (33001, 256), (35000, 100), (32768, 64), (33333, 7)]:
        X = rng.integers(-50, 50, (rows, cols)).astype(np.float32)  # many ties
        dX = F.from_numpy(X)
        np.testing.assert_array_equal(F.max(dX).numpy()[:, 0], X.max(axis=1))
        np.testing.assert_array_equal(F.min(dX).numpy()[:, 0], X.min(axis=1))
        np.testing.assert_array_equal(F.argmax(dX).numpy()[:, 0], X.argmax(axis=1))
        np.testing.assert_array_equal(F.argmin(dX).numpy()[:, 0], X.argmin(axis=1))


def test_select_full_size(gpu):
    """(8192, 8192): every row's maximum, and that x[argmax] is that maximum."""
    F = gpu.functional
    rng = np.random.Generator(np.random.PCG64(9))
    x = rng.standard_normal((8192, 8192)).astype(np.float32)
    dx = F.from_numpy(x)
    mx = F.max(dx).numpy().ravel()
    assert_bit_equal(mx, x.max(axis=1), "row max")
    am = F.argmax(dx).numpy().ravel()
    assert np.array_equal(x[np.arange(8192), am], mx)
    assert np.array_equal(am, x.argmax(axis=1))


def test_fused_activations_match_their_node_recipes(gpu):
    """!relu, !leaky-relu and !sigmoid as single kernels against the node
    sequences of nn/activation.lisp:11-92 run one node at a time: bit-identical
    (the kernels perform the same binary32 operations in the same order), on
    random data, special values and a strided view; sigmoid also within 2 ulp of
    float64."""
    W = gpu
    F = W.functional
    rng = np.random.default_rng(41)
    x = (rng.standard_normal(100003) * 4).astype(np.float32)
    x[:16] = [0.0, -0.0, np.inf, -np.inf, np.nan, 1e-45, -1e-45, 88.0, -88.0, 104.0, -104.0, 1e30, -1e30, 1.0, -1.0, 20.0]
    dx = F.from_numpy(x)
    pairs = [(F.relu_fused, F.relu), (F.sigmoid_fused, F.sigmoid),
             (lambda t: F.leaky_relu_fused(t, 0.2), lambda t: F.leaky_relu(t, 0.2))]
    for view in (dx, F.reshape(F.from_numpy(x[:99840]), 312, 320).view((3, 300, 2), (5, 305, 3))):
        for fused, recipe in pairs:
            a, b = fused(view).numpy(), recipe(view).numpy()
            nan = np.isnan(b)  # a NaN stays a NaN; its sign bit is not part of the contract
            assert np.array_equal(np.isnan(a), nan)
            np.testing.assert_array_equal(a[~nan].view(np.uint32), b[~nan].view(np.uint32))
    s = F.sigmoid_fused(dx).numpy()[16:]
    truth = (1.0 / (1.0 + np.exp(-x[16:].astype(np.float64)))).astype(np.float32)
    assert np.abs(s.view(np.int32).astype(np.int64) - truth.view(np.int32).astype(np.int64)).max() <= 2
    assert np.array_equal(F.relu_fused(dx).numpy()[16:], np.maximum(x[16:], 0.0))
