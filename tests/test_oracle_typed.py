"""The oracle's restatement of the non-:float arithmetic kernels against the
golden vectors of the compiled reference (tests/golden/typed_kernels.npz, from
waffe2_d*, waffe2_{i32,i16,i8,u32,u16,u8}* of cl-waffe2-simd.c) and against
closed forms that a plausible mistake breaks: numpy's wrap-around integer
arithmetic, binary64 arithmetic for the vector body of the :double kernels and
the binary32 round trip of their remainder loop."""
import os

import numpy as np
import pytest

GOLD = os.path.join(os.path.dirname(__file__), "golden", "typed_kernels.npz")
OPS = ("add", "sub", "mul", "div", "copy")


@pytest.fixture(scope="module")
def gold():
    return np.load(GOLD)


def _cases(gold, key):
    for n, incx, incy, start, size in gold[key + "_cases"]:
        yield int(n), int(incx), int(incy), slice(int(start), int(start + size))


@pytest.mark.parametrize("dtype", ["double", "int32", "uint32", "int16", "uint16", "int8", "uint8"])
def test_oracle_matches_reference_goldens(O, gold, dtype):
    checked = 0
    for op in OPS:
        key = f"{dtype}_{op}"
        if key + "_x" not in gold:
            continue
        for n, incx, incy, sl in _cases(gold, key):
            got = gold[key + "_x"][sl].copy()
            O.binary_typed_1d(dtype, op, n, got, incx, gold[key + "_y"][sl].copy(), incy)
            np.testing.assert_array_equal(got.view(np.uint8), gold[key + "_out"][sl].view(np.uint8),
                                          err_msg=f"{key} n={n} incx={incx} incy={incy}")
            checked += 1
    for n, incx, _, sl in _cases(gold, f"{dtype}_inv"):
        got = gold[f"{dtype}_inv_x"][sl].copy()
        O.inv_typed_1d(dtype, n, got, incx)
        np.testing.assert_array_equal(got.view(np.uint8), gold[f"{dtype}_inv_out"][sl].view(np.uint8))
        checked += 1
    assert checked > 100


@pytest.mark.parametrize("dtype", ["int32", "uint32", "int16", "uint16", "int8", "uint8"])
def test_integer_kernels_are_c_arithmetic(O, dtype):
    """Closed form: two's-complement wrap-around through int64 arithmetic;
    division truncates toward zero."""
    npt = O.DTYPES[dtype][1]
    info = np.iinfo(npt)
    rng = np.random.default_rng(5)
    n = 1000
    x = rng.integers(info.min, info.max, n, endpoint=True).astype(npt)
    y = rng.integers(info.min, info.max, n, endpoint=True).astype(npt)
    y[y == 0] = 7
    x[x == info.min] = info.min + 1
    x64, y64 = x.astype(np.int64), y.astype(np.int64)
    want = {"add": x64 + y64, "sub": x64 - y64, "mul": x64 * y64,
            "div": np.trunc(x64 / y64).astype(np.int64)}
    for op, w in want.items():
        got = x.copy()
        O.binary_typed_1d(dtype, op, n, got, 1, y, 1)
        bits = 8 * np.dtype(npt).itemsize
        wrapped = (w & ((1 << bits) - 1)).astype(np.uint64).astype(np.dtype(f"uint{bits}")).view(npt)
        np.testing.assert_array_equal(got, wrapped, err_msg=f"{dtype} {op}")


def test_double_kernels_round_their_remainder_through_binary32(O):
    """Vector body ((n / 4) * 4 elements when incx >= 1): binary64; the rest,
    and everything when incx == 0: (double)(float)(x op y)."""
    rng = np.random.default_rng(6)
    n = 23
    x = rng.standard_normal(n * 2)
    y = rng.standard_normal(n * 2)
    for incx in (1, 2):
        got = x.copy()
        O.binary_typed_1d("double", "mul", n, got, incx, y, 1)
        idx = np.arange(n) * incx
        exact = x[idx] * y[:n]
        want = np.where(np.arange(n) < (n // 4) * 4, exact, exact.astype(np.float32).astype(np.float64))
        np.testing.assert_array_equal(got[idx], want)
        assert np.any(got[idx][20:] != exact[20:])  # the quirk is visible on random data
    acc = np.array([0.25])
    O.binary_typed_1d("double", "add", n, acc, 0, y, 1)
    want = np.float64(0.25)
    for v in y[:n]:
        want = np.float64(np.float32(want + v))
    assert acc[0] == want
