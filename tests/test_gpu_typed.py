"""GPU parity of the arithmetic / move kernels for :double and the integer
dtypes: bit-exact against the golden vectors of the compiled reference
(tests/golden/typed_kernels.npz) and the oracle on larger seeded inputs through
the 1-D entry points; numpy closed forms through the node layer (N-D views)."""
import ctypes as C
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

GOLD = os.path.join(os.path.dirname(__file__), "golden", "typed_kernels.npz")
DTYPES = ["double", "int32", "uint32", "int16", "uint16", "int8", "uint8"]
OPS = {"add": 0, "sub": 1, "mul": 2, "div": 3, "copy": 4}


def _bits(a):
    return np.ascontiguousarray(a).view(np.uint8)


@pytest.mark.parametrize("dtype", DTYPES)
def test_1d_entry_points_against_reference_goldens(gpu, O, dtype):
    W = gpu
    lib = W.lib.get()
    gold = np.load(GOLD)
    code = W.lib.DTYPE_CODES[dtype]
    size = np.dtype(O.DTYPES[dtype][1]).itemsize
    for op, opcode in OPS.items():
        key = f"{dtype}_{op}"
        if key + "_x" not in gold:
            continue
        for n, incx, incy, start, length in gold[key + "_cases"]:
            sl = slice(int(start), int(start + length))
            dx = W.HIPTensor.from_numpy(gold[key + "_x"][sl], dtype=dtype)
            dy = W.HIPTensor.from_numpy(gold[key + "_y"][sl], dtype=dtype)
            W.lib.check(lib.wf2hip_binary_1d_typed(code, opcode, int(n), C.c_void_p(dx.ptr), int(incx),
                                                   C.c_void_p(dy.ptr), int(incy)))
            np.testing.assert_array_equal(_bits(dx.numpy()), _bits(gold[key + "_out"][sl]),
                                          err_msg=f"{key} n={n} incx={incx} incy={incy}")
    for n, incx, _, start, length in gold[f"{dtype}_inv_cases"]:
        sl = slice(int(start), int(start + length))
        dx = W.HIPTensor.from_numpy(gold[f"{dtype}_inv_x"][sl], dtype=dtype)
        W.lib.check(lib.wf2hip_inv_1d_typed(code, int(n), C.c_void_p(dx.ptr), int(incx)))
        np.testing.assert_array_equal(_bits(dx.numpy()), _bits(gold[f"{dtype}_inv_out"][sl]))
    assert size in (1, 2, 4, 8)


@pytest.mark.parametrize("dtype", DTYPES)
def test_1d_entry_points_against_oracle_at_size(gpu, O, dtype):
    """Sizes that reach the 16-byte vector kernel, its scalar remainder, unaligned
    starts and every increment regime; named wrappers (wf2hip_dadd ...) included."""
    W = gpu
    lib = W.lib.get()
    code, npt, prefix = O.DTYPES[dtype]
    rng = np.random.default_rng(31 + code)
    item = np.dtype(npt).itemsize

    def draw(size, op):
        if dtype == "double":
            return rng.standard_normal(size), rng.uniform(0.5, 2.0, size) * rng.choice([-1.0, 1.0], size)
        info = np.iinfo(npt)
        x = rng.integers(info.min, info.max, size, endpoint=True).astype(npt)
        y = rng.integers(info.min, info.max, size, endpoint=True).astype(npt)
        if op == "div":
            y = np.where(rng.random(size) < 0.6, rng.integers(1, 9, size).astype(npt), y).astype(npt)
            y[y == 0] = 5
            x[x == info.min] = info.max
        return x, y

    for op, opcode in OPS.items():
        for n, incx, incy, offx, offy in [(100003, 1, 1, 0, 0), (65536, 1, 0, 0, 0), (40001, 1, 1, 1, 0),
                                          (30000, 2, 1, 0, 3), (30000, 1, 3, 0, 0), (999, 3, 2, 2, 1),
                                          (777, 0, 1, 5, 0), (0, 1, 1, 0, 0)]:
            if incx == 0 and dtype != "double" and op in ("mul",):
                pass  # wrap-around products are fine for integers
            size = max(n, 1) * 3 + 8
            x, y = draw(size, op)
            x, y = x.astype(npt), y.astype(npt)
            if incx == 0 and op == "div" and dtype != "double":
                y[:] = 1 + (np.arange(size) % 3)
            want = x.copy()
            O.binary_typed_1d(dtype, op, n, want, incx, y, incy, offx=offx, offy=offy)
            dx, dy = W.HIPTensor.from_numpy(x, dtype=dtype), W.HIPTensor.from_numpy(y, dtype=dtype)
            px, py = C.c_void_p(dx.ptr + item * offx), C.c_void_p(dy.ptr + item * offy)
            if op == "copy" and dtype == "double":
                fn = lib.wf2hip_dcopy
                fn.argtypes = [C.c_long, C.c_void_p, C.c_long, C.c_void_p, C.c_long]
                W.lib.check(fn(n, py, incy, px, incx))
            else:
                fn = getattr(lib, f"wf2hip_{prefix}{op}")
                fn.argtypes = [C.c_long, C.c_void_p, C.c_long, C.c_void_p, C.c_long]
                fn.restype = C.c_int
                W.lib.check(fn(n, px, incx, py, incy))
            np.testing.assert_array_equal(_bits(dx.numpy()), _bits(want),
                                          err_msg=f"{dtype} {op} n={n} incx={incx} incy={incy} off=({offx},{offy})")


@pytest.mark.parametrize("dtype", DTYPES)
def test_nodes_on_views(gpu, dtype):
    """AddNode ... MoveTensorNode through the node layer on N-D views (slices,
    steps, broadcasts, permutes): numpy closed form (binary64 arithmetic for
    :double -- the N-D entry has no per-call remainder --, wrap-around for ints)."""
    W = gpu
    F = W.functional
    from importlib import import_module
    npt = import_module("cl-waffe2_amd.tensor").DTYPES[dtype]
    rng = np.random.default_rng(77)

    def draw(shape, nonzero=False):
        if dtype == "double":
            a = rng.standard_normal(shape)
            return a + np.sign(a) if nonzero else a
        info = np.iinfo(npt)
        if nonzero:
            return rng.integers(1, 9, shape).astype(npt)
        return rng.integers(info.min // 2, info.max // 2, shape, endpoint=True).astype(npt)

    A = draw((12, 40, 34))
    dA = F.from_numpy(A, dtype=dtype)
    with np.errstate(over="ignore"):
        # contiguous, both operands full
        B = draw(A.shape)
        got = F.add(dA, F.from_numpy(B, dtype=dtype))
        np.testing.assert_array_equal(got.numpy(), (A + B).astype(npt))
        # slices with steps against a row broadcast
        v = dA.view((2, 10), (0, 40, 3), (1, 33, 2))
        R = draw((1, 1, 16))
        x = F.copy(v)
        assert x.dtype == dtype and x.shape == [8, 13, 16]  # a range holds floor((to - from) / step) elements
        F.sub_(x, F.from_numpy(R, dtype=dtype).view((":broadcast", 8), (":broadcast", 13), True))
        np.testing.assert_array_equal(x.numpy(), (A[2:10, 0:40:3, 1:33:2][:, :13] - R).astype(npt))
        # permuted source, scalar operand, division by a non-zero tensor
        p = F.copy(dA.permute(2, 0, 1))
        np.testing.assert_array_equal(p.numpy(), np.transpose(A, (2, 0, 1)))
        s = F.mul(dA, 3)
        np.testing.assert_array_equal(s.numpy(), (A * npt(3)).astype(npt))
        D = draw(A.shape, nonzero=True)
        q = F.div(dA, F.from_numpy(D, dtype=dtype))
        want = A / D if dtype == "double" else np.trunc(A.astype(np.float64) / D).astype(npt)
        np.testing.assert_array_equal(q.numpy(), want)


@pytest.mark.parametrize("dtype", DTYPES)
def test_accumulation_into_broadcast_destinations(gpu, dtype):
    """!sum as the reference composes it (zero-fill, (:broadcast n) view, AddNode):
    integer sums wrap modulo 2^bits in any order, so numpy's wrapped sum is the exact
    answer; :double within 1e-13 relative to the sum of magnitudes.  SubNode into a
    broadcast destination follows the sequential order (exact for integers)."""
    W = gpu
    F = W.functional
    from importlib import import_module
    npt = import_module("cl-waffe2_amd.tensor").DTYPES[dtype]
    rng = np.random.default_rng(91)
    if dtype == "double":
        A = rng.standard_normal((7, 300, 41))
    else:
        info = np.iinfo(npt)
        A = rng.integers(info.min, info.max, (7, 300, 41), endpoint=True).astype(npt)
    dA = F.from_numpy(A, dtype=dtype)

    def check(got, axis):
        want = A.sum(axis=axis, keepdims=True, dtype=npt if dtype != "double" else np.float64)
        assert got.dtype == dtype and list(got.shape) == list(want.shape)
        if dtype == "double":
            scale = np.abs(A).sum(axis=axis, keepdims=True)
            assert np.max(np.abs(got.numpy() - want) / scale) < 1e-13
        else:
            np.testing.assert_array_equal(got.numpy(), want)

    with np.errstate(over="ignore"):
        check(F.sum(dA, axis=2), 2)
        check(F.sum(dA, axis=0), 0)
        check(F.sum(dA, axis=(0, 2)), (0, 2))
        check(F.sum(dA), (0, 1, 2))
        # a strided window
        v = dA.view((1, 6), (0, 300, 7), (2, 40, 3))
        W_ = A[1:6, 0:300:7, 2:40:3][:, :42, :12]
        got = F.sum(v, axis=1)
        want = W_.sum(axis=1, keepdims=True, dtype=npt if dtype != "double" else np.float64)
        if dtype == "double":
            assert np.max(np.abs(got.numpy() - want)) < 1e-11
        else:
            np.testing.assert_array_equal(got.numpy(), want)
        # long reductions into few destinations (the split kernel): a full sum and two column sums
        big = (rng.standard_normal((2, 150001)) if dtype == "double"
               else rng.integers(info.min, info.max, (2, 150001), endpoint=True).astype(npt))
        dbig = F.from_numpy(big, dtype=dtype)
        for axis in ((0, 1), 1):
            got = F.sum(dbig, axis=axis)
            want = big.sum(axis=axis, keepdims=True, dtype=npt if dtype != "double" else np.float64)
            if dtype == "double":
                assert np.max(np.abs(got.numpy() - want)) < 1e-9
            else:
                np.testing.assert_array_equal(got.numpy(), want)
        # sums over the leading axes with a contiguous kept axis of 64 columns or more (column form)
        for shape, axis in (((700, 130), 0), ((33, 40, 260), (0, 1)), ((5000, 64), 0)):
            Z = (rng.standard_normal(shape) if dtype == "double"
                 else rng.integers(info.min, info.max, shape, endpoint=True).astype(npt))
            got = F.sum(F.from_numpy(Z, dtype=dtype), axis=axis)
            want = Z.sum(axis=axis, keepdims=True, dtype=npt if dtype != "double" else np.float64)
            if dtype == "double":
                assert np.max(np.abs(got.numpy() - want)) < 1e-9
            else:
                np.testing.assert_array_equal(got.numpy(), want)
        # x[0, j] <- x[0, j] - sum_i y[i, j], sequentially
        base = A[0, 0:1, :].copy()
        dst = F.from_numpy(base, dtype=dtype).view((":broadcast", 300), True)
        F.sub_(dst, F.from_numpy(A[1], dtype=dtype))
        if dtype == "double":
            want = base - A[1].sum(axis=0, keepdims=True)
            assert np.max(np.abs(dst.storage_numpy().reshape(1, 41) - want)) < 1e-10
        else:
            want = (base.astype(np.int64) - A[1].astype(np.int64).sum(axis=0, keepdims=True)).astype(npt)
            np.testing.assert_array_equal(dst.storage_numpy().reshape(1, 41), want)


@pytest.mark.parametrize("dtype", ["double", "int32", "uint8"])
def test_1d_entry_refuses_overlapping_runs(gpu, dtype):
    """x <- x op y reads y while other lanes write x: two different runs over one buffer
    are refused (as the N-D entry point refuses them); a stride-0 source in a buffer of
    its own, the way a non-:float tensor is filled with its initial element, is fine, and
    so is the same run on both sides (x <- x + x)."""
    W = gpu
    lib = W.lib.get()
    code = W.lib.DTYPE_CODES[dtype]
    npt = {"double": np.float64, "int32": np.int32, "uint8": np.uint8}[dtype]
    n = 5000
    dx = W.HIPTensor.from_numpy(np.arange(n) % 50, dtype=dtype)
    for op in (W.lib.MOVE, W.lib.ADD):
        rc = lib.wf2hip_binary_1d_typed(code, op, n, C.c_void_p(dx.ptr), 1, C.c_void_p(dx.ptr), 0)
        assert rc == W.lib.EOVERLAP
    item = np.dtype(npt).itemsize
    assert lib.wf2hip_binary_1d_typed(code, W.lib.ADD, n - 1, C.c_void_p(dx.ptr), 1,
                                      C.c_void_p(dx.ptr + item), 1) == W.lib.EOVERLAP
    one = W.HIPTensor.from_numpy(np.array([7]), dtype=dtype)
    W.lib.check(lib.wf2hip_binary_1d_typed(code, W.lib.MOVE, n, C.c_void_p(dx.ptr), 1, C.c_void_p(one.ptr), 0))
    assert np.all(dx.numpy() == 7)
    W.lib.check(lib.wf2hip_binary_1d_typed(code, W.lib.ADD, n, C.c_void_p(dx.ptr), 1, C.c_void_p(dx.ptr), 1))
    assert np.all(dx.numpy() == 14)


@pytest.mark.parametrize("dtype", ["double", "int32", "uint32", "int16", "uint16", "int8", "uint8"])
@pytest.mark.parametrize("seed", range(6))
def test_typed_random_permuted_passes(gpu, dtype, seed):
    """Copies out of and into permuted windows and accumulating passes over them on every element type, random
    ranks, extents and axis orders: the tiled transposing kernel and the element-per-lane kernel against
    numpy's indexing (integer sums wrap, as the reference's C loops do); bit-exact."""
    F = gpu.functional
    np_dtype = {"double": np.float64, "int32": np.int32, "uint32": np.uint32, "int16": np.int16, "uint16": np.uint16,
                "int8": np.int8, "uint8": np.uint8}[dtype]
    rng = np.random.default_rng(77 * seed + len(dtype))
    extents = [1, 2, 3, 15, 16, 17, 63, 64, 65, 100, 257, 300]
    rank = int(rng.integers(2, 5))
    while True:
        shape = [int(rng.choice(extents)) for _ in range(rank)]
        if np.prod(shape) <= 300000:
            break
    perm = tuple(int(p) for p in rng.permutation(rank))

    def draw(sh):
        if dtype == "double":
            return rng.standard_normal(sh)
        info = np.iinfo(np_dtype)
        return rng.integers(info.min, int(info.max) + 1, sh).astype(np_dtype)

    x = draw(shape)
    dx = F.from_numpy(x, dtype=dtype)
    axis = int(rng.integers(0, rank))
    lo = 1 if shape[axis] > 2 else 0
    subs = [True] * rank
    subs[axis] = (lo, shape[axis])
    index = tuple(slice(lo, None) if a == axis else slice(None) for a in range(rank))
    xv, dv = x[index], dx.view(*subs)
    what = f"{dtype} {shape} {perm} axis {axis} from {lo}"
    np.testing.assert_array_equal(F.copy(dv.permute(*perm)).numpy(), xv.transpose(perm), err_msg="copy " + what)
    y = draw(xv.transpose(perm).shape)
    dy = F.from_numpy(y, dtype=dtype)
    back = np.argsort(perm)
    want = x.copy()
    with np.errstate(over="ignore"):
        want[index] = xv + y.transpose(back)
    F.add_(dv.permute(*perm), dy)
    np.testing.assert_array_equal(dx.numpy(), want, err_msg="accumulate into the permuted window, " + what)
    with np.errstate(over="ignore"):
        want2 = y - want[index].transpose(perm)
    F.sub_(dy, dv.permute(*perm))
    np.testing.assert_array_equal(dy.numpy(), want2, err_msg="subtract a permuted window, " + what)


@pytest.mark.parametrize("dtype", ["int16", "uint16", "int8", "uint8"])
@pytest.mark.parametrize("seed", range(5))
def test_sliced_rows_of_the_narrow_types(gpu, dtype, seed):
    """Windows with stride 1 along the last axis (a slice of every row, of several leading axes, a row broadcast
    as the other operand): rows of 64 bytes and more run 16 bytes per lane, whatever byte the rows of either
    side start on -- every start and length modulo 16 appears; bit-exact against numpy (sums wrap, quotients
    truncate, as in the reference's loops, cl-waffe2-simd.c:252-288)."""
    F = gpu.functional
    npt = {"int16": np.int16, "uint16": np.uint16, "int8": np.int8, "uint8": np.uint8}[dtype]
    rng = np.random.default_rng(1000 * seed + len(dtype) + npt().itemsize)
    info = np.iinfo(npt)

    def draw(sh, nonzero=False):
        if nonzero:
            return rng.integers(1, 12, sh).astype(npt)
        return rng.integers(info.min, int(info.max) + 1, sh).astype(npt)

    for case in range(6):
        rank = int(rng.integers(2, 5))
        width = int(rng.choice([70, 129, 300, 1024, 4099, 70000 if rank == 2 else 513]))
        shape = [int(rng.integers(2, 7)) for _ in range(rank - 1)] + [width]
        lo = int(rng.integers(0, 19))
        hi = width - int(rng.integers(0, 19))
        lead_lo = int(rng.integers(0, 2))
        x, y = draw(shape), draw(shape)
        dx, dy = F.from_numpy(x, dtype=dtype), F.from_numpy(y, dtype=dtype)
        lo_y = int(rng.integers(0, 19))  # the other side starts on another byte
        lo_y = min(lo_y, width - (hi - lo))
        subs_x = [(lead_lo, shape[0])] + [True] * (rank - 2) + [(lo, hi)]
        subs_y = [(lead_lo, shape[0])] + [True] * (rank - 2) + [(lo_y, lo_y + hi - lo)]
        ix = (slice(lead_lo, None),) + (slice(None),) * (rank - 2) + (slice(lo, hi),)
        iy = (slice(lead_lo, None),) + (slice(None),) * (rank - 2) + (slice(lo_y, lo_y + hi - lo),)
        what = f"{dtype} {shape} x[{lo}:{hi}] y[{lo_y}:] lead {lead_lo}"
        with np.errstate(over="ignore"):
            want = x.copy()
            want[ix] = x[ix] + y[iy]
            F.add_(dx.view(*subs_x), dy.view(*subs_y))
            np.testing.assert_array_equal(dx.numpy(), want, err_msg="add " + what)
            want[ix] = want[ix] * y[iy]
            F.mul_(dx.view(*subs_x), dy.view(*subs_y))
            np.testing.assert_array_equal(dx.numpy(), want, err_msg="mul " + what)
            want2 = y.copy()
            want2[iy] = y[iy] - want[ix]
            F.sub_(dy.view(*subs_y), dx.view(*subs_x))
            np.testing.assert_array_equal(dy.numpy(), want2, err_msg="sub " + what)
        d = draw(shape, nonzero=True)
        dd = F.from_numpy(d, dtype=dtype)
        F.div_(dx.view(*subs_x), dd.view(*subs_y))
        want[ix] = np.trunc(want[ix].astype(np.float64) / d[iy]).astype(npt)
        np.testing.assert_array_equal(dx.numpy(), want, err_msg="div " + what)
        # a copy out of the window, and one row added to every row of it
        np.testing.assert_array_equal(F.copy(dx.view(*subs_x)).numpy(), want[ix], err_msg="copy " + what)
        row = draw((hi - lo,))
        bview = F.from_numpy(row.reshape((1,) * (rank - 1) + (-1,)), dtype=dtype).view(
            *([(":broadcast", shape[0] - lead_lo)] + [(":broadcast", n) for n in shape[1:-1]] + [True]))
        with np.errstate(over="ignore"):
            want[ix] = want[ix] + row
        F.add_(dx.view(*subs_x), bview)
        np.testing.assert_array_equal(dx.numpy(), want, err_msg="row broadcast " + what)
