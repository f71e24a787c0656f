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
    """2^26 elements through the streaming kernel; ReLU at BASELINE size via the
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
