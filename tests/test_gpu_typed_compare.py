"""GPU parity of the compare / where kernels on :double and the integer types:
bit-exact against the golden vectors of the compiled reference
(tests/golden/typed_compare_kernels.npz) and the oracle at larger sizes through the
1-D entry points (wf2hip_<prefix>{eq,...} and ..._scal), numpy closed forms through
the node layer (N-D views, the element type's own order)."""
import ctypes as C
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

GOLD = os.path.join(os.path.dirname(__file__), "golden", "typed_compare_kernels.npz")
DTYPES = ["double", "int32", "uint32", "int16", "uint16", "int8", "uint8"]
CTYPES = {"double": C.c_double, "int32": C.c_int32, "uint32": C.c_uint32, "int16": C.c_int16,
          "uint16": C.c_uint16, "int8": C.c_int8, "uint8": C.c_uint8}


def call_1d(W, O, dtype, op, n, dx, incx, y, incy, dout, inco, then, els, offo=0):
    lib = W.lib.get()
    prefix = O.DTYPES[dtype][2]
    ct = CTYPES[dtype]
    item = dx.itemsize
    if isinstance(y, W.HIPTensor):
        fn = getattr(lib, f"wf2hip_{prefix}{op}")
        W.lib.check(fn(n, C.c_void_p(dx.ptr), incx, C.c_void_p(y.ptr), incy, C.c_void_p(dout.ptr + item * offo), inco,
                       ct(then), ct(els)))
    else:
        fn = getattr(lib, f"wf2hip_{prefix}{op}_scal")
        W.lib.check(fn(n, C.c_void_p(dx.ptr), incx, C.c_void_p(dout.ptr + item * offo), inco, ct(y), ct(then), ct(els)))


@pytest.mark.parametrize("dtype", DTYPES)
def test_1d_entry_points_against_reference_goldens(gpu, O, dtype):
    W = gpu
    gold = np.load(GOLD)
    then, els = (1.5, -0.25) if dtype == "double" else (3, 5)
    for op, n, incx, incy, inco, scal, start, size in gold[f"{dtype}_cmp_cases"]:
        sl = slice(int(start), int(start + size))
        x, y = gold[f"{dtype}_cmp_x"][sl], gold[f"{dtype}_cmp_y"][sl]
        dx = W.HIPTensor.from_numpy(x, dtype=dtype)
        dout = W.HIPTensor.from_numpy(np.full(x.size, 7, x.dtype), dtype=dtype)
        yy = y[0].item() if scal else W.HIPTensor.from_numpy(y, dtype=dtype)
        call_1d(W, O, dtype, O.CMP_OPS[int(op)], int(n), dx, int(incx), yy, int(incy), dout, int(inco), then, els)
        np.testing.assert_array_equal(dout.numpy().view(np.uint8), gold[f"{dtype}_cmp_out"][sl].view(np.uint8),
                                      err_msg=f"{dtype} {O.CMP_OPS[int(op)]} n={n} inc=({incx},{incy},{inco}) scal={scal}")


@pytest.mark.parametrize("dtype", DTYPES)
def test_1d_entry_points_against_oracle_at_size(gpu, O, dtype):
    """Sizes that reach the 16-byte vector kernel and its remainder, unit and other
    increments, a stride-0 and a backwards `out`; values on both sides of the sign
    bit so that the signed blocks of the unsigned types show."""
    W = gpu
    npt = O.DTYPES[dtype][1]
    rng = np.random.default_rng(41)
    for n, incx, incy, inco in [(100003, 1, 1, 1), (65536, 1, 1, 1), (4099, 2, 1, 1), (3001, 1, 3, 2),
                                (777, 1, 1, 0), (515, 3, 2, -1), (31, 1, 1, 1), (0, 1, 1, 1)]:
        size = max(n, 1) * 3 + 8
        if dtype == "double":
            x = rng.integers(-3, 4, size).astype(npt)
            y = rng.integers(-3, 4, size).astype(npt)
            x[rng.random(size) < 0.05] = np.nan
        else:
            info = np.iinfo(npt)
            x = rng.integers(info.min, info.max, size, endpoint=True).astype(npt)
            y = np.where(rng.random(size) < 0.3, x, rng.integers(info.min, info.max, size, endpoint=True)).astype(npt)
        offo = (n - 1) * -inco if inco < 0 and n > 0 else 0
        for op in O.CMP_OPS:
            for scal in (False, True):
                want = np.full(size, 9, npt)
                O.cmp_typed_1d(dtype, op, n, x, incx, y[2].item() if scal else y, incy, want, inco, 4, 6, offo=offo)
                dx = W.HIPTensor.from_numpy(x, dtype=dtype)
                dout = W.HIPTensor.from_numpy(np.full(size, 9, npt), dtype=dtype)
                yy = y[2].item() if scal else W.HIPTensor.from_numpy(y, dtype=dtype)
                call_1d(W, O, dtype, op, n, dx, incx, yy, incy, dout, inco, 4, 6, offo=offo)
                np.testing.assert_array_equal(dout.numpy(), want,
                                              err_msg=f"{dtype} {op} n={n} inc=({incx},{incy},{inco}) scal={scal}")


@pytest.mark.parametrize("dtype", DTYPES)
def test_nodes_on_views(gpu, dtype):
    """Compare-Operation-Node / Where-Operation-Node through the node layer on N-D
    views: numpy in the element type's own order."""
    W = gpu
    F = W.functional
    from importlib import import_module
    npt = import_module("cl-waffe2_amd.tensor").DTYPES[dtype]
    rng = np.random.default_rng(78)

    def draw(shape):
        if dtype == "double":
            a = rng.integers(-3, 4, shape).astype(npt)
            a[rng.random(shape) < 0.05] = np.nan
            return a
        info = np.iinfo(npt)
        return rng.integers(info.min, info.max, shape, endpoint=True).astype(npt)

    A, B = draw((6, 40, 34)), draw((6, 40, 34))
    B = np.where(rng.random(B.shape) < 0.3, A, B)
    dA, dB = F.from_numpy(A, dtype=dtype), F.from_numpy(B, dtype=dtype)
    scal = A[1, 2, 3].item() if dtype != "double" else 1.0
    ops = {"<": np.less, "<=": np.less_equal, ">": np.greater, ">=": np.greater_equal, "=": np.equal}
    for cond, fn in ops.items():
        got = F.compare(dA, dB, cond, 2, 7)
        assert got.dtype == dtype
        np.testing.assert_array_equal(got.numpy(), np.where(fn(A, B), 2, 7).astype(npt), err_msg=cond)
        got = F.where(dA, cond, scal, 1, 0)
        np.testing.assert_array_equal(got.numpy(), np.where(fn(A, npt(scal)), 1, 0).astype(npt), err_msg=cond)
        # sliced / permuted operands, a row-broadcast right-hand side
        va, vb = dA.view((1, 5), (0, 40, 3), (1, 33, 2)), dB.permute(0, 2, 1).view((1, 5), (1, 33, 2), (0, 40, 3)).permute(0, 2, 1)
        got = F.compare(va, vb, cond, 1, 0)
        np.testing.assert_array_equal(got.numpy(), np.where(fn(A[1:5, 0:40:3, 1:33:2][:, :13], B[1:5, 0:40:3, 1:33:2][:, :13]), 1, 0).astype(npt))
        row = F.from_numpy(B[0:1, 0:1, :], dtype=dtype).view(True, (":broadcast", 40), True)
        got = F.compare(dA.view(2, True, True), row, cond, 1, 0)
        np.testing.assert_array_equal(got.numpy(), np.where(fn(A[2:3], B[0:1, 0:1, :]), 1, 0).astype(npt))


EXTREME_GOLD = os.path.join(os.path.dirname(__file__), "golden", "typed_extreme_kernels.npz")


@pytest.mark.parametrize("dtype", DTYPES)
def test_extremes_against_goldens_and_oracle(gpu, O, dtype):
    """wf2hip_<prefix>{max,min}: the compiled reference's goldens, then the oracle on
    runs long enough for the split kernel, unit and other increments."""
    W = gpu
    lib = W.lib.get()
    npt, prefix = O.DTYPES[dtype][1], O.DTYPES[dtype][2]
    gold = np.load(EXTREME_GOLD)

    def run(op, n, x, incx, off=0):
        dx = W.HIPTensor.from_numpy(x, dtype=dtype)
        dout = W.HIPTensor.from_numpy(np.zeros(1, npt), dtype=dtype)
        W.lib.check(getattr(lib, f"wf2hip_{prefix}{op}")(n, C.c_void_p(dx.ptr + dx.itemsize * off), incx,
                                                         C.c_void_p(dout.ptr)))
        return dout.numpy()[0]

    for k, (op, n, incx, start, size) in enumerate(gold[f"{dtype}_extreme_cases"]):
        x = gold[f"{dtype}_extreme_x"][int(start):int(start + size)]
        assert run(("max", "min")[int(op)], int(n), x, int(incx)) == gold[f"{dtype}_extreme_out"][k]
    rng = np.random.default_rng(29)
    for n, incx, off in [(1, 1, 0), (100, 1, 1), (5000, 1, 0), (300001, 1, 4), (70001, 3, 2)]:
        size = n * incx + off + 1
        if dtype == "double":
            x = rng.standard_normal(size)
        else:
            info = np.iinfo(npt)
            x = rng.integers(info.min, info.max, size, endpoint=True).astype(npt)
        for op in ("max", "min"):
            assert run(op, n, x, incx, off) == O.extreme_typed_1d(dtype, op, n, x, incx, offx=off), (dtype, op, n, incx)


@pytest.mark.parametrize("dtype", DTYPES)
def test_max_min_nodes(gpu, dtype):
    """!max / !min on every dtype, !argmax / !argmin on :double (first occurrence),
    numpy closed forms; index nodes on integer tensors have no device kernel."""
    W = gpu
    F = W.functional
    from importlib import import_module
    npt = import_module("cl-waffe2_amd.tensor").DTYPES[dtype]
    rng = np.random.default_rng(83)
    if dtype == "double":
        A = rng.integers(-50, 50, (37, 1000)).astype(npt) / 4
    else:
        info = np.iinfo(npt)
        A = rng.integers(info.min, info.max, (37, 1000), endpoint=True).astype(npt)
    dA = F.from_numpy(A, dtype=dtype)
    got = F.max(dA)
    assert got.dtype == dtype and got.shape == [37, 1]
    np.testing.assert_array_equal(got.numpy()[:, 0], A.max(axis=1))
    np.testing.assert_array_equal(F.min(dA).numpy()[:, 0], A.min(axis=1))
    # strided rows: every second column of a window
    v = dA.view((3, 30), (1, 999, 2))
    np.testing.assert_array_equal(F.max(v).numpy()[:, 0], A[3:30, 1:999:2].max(axis=1))
    # the whole tensor as one run
    np.testing.assert_array_equal(F.min(dA, axis=2).numpy().ravel(), [A.min()])
    if dtype == "double":
        np.testing.assert_array_equal(F.argmax(dA).numpy()[:, 0], A.argmax(axis=1))
        np.testing.assert_array_equal(F.argmin(dA).numpy()[:, 0], A.argmin(axis=1))
    else:
        with pytest.raises(W.nodes.NodeNotFound):
            F.argmax(dA)
