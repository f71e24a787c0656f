"""The oracle's restatement of the compare / where kernels on :double and the
integer types against the golden vectors of the compiled reference
(tests/golden/typed_compare_kernels.npz, from waffe2_<prefix>{eq,lt,le,gt,ge} and
..._scal of cl-waffe2-simd.c) and against numpy closed forms: the element type's own
order in the scalar loop, the signed order in the 32-byte blocks of the unsigned
types, ordered predicates (false on NaN) for :double.

The reference builds strided integer lanes by indexing a 4-lane vector up to lane
31 (cl-waffe2-simd.c:54-107, 119-141), so its block part is undefined for the integer
types unless every increment is 1, and the compiled reference faults or spins on
most 8- and 16-bit cases with inco >= 1.  The fixture holds the cases that are
defined and ran; the rest of the oracle's behaviour there follows the source text
and is pinned by the closed forms only."""
import os

import numpy as np
import pytest

GOLD = os.path.join(os.path.dirname(__file__), "golden", "typed_compare_kernels.npz")
DTYPES = ["double", "int32", "uint32", "int16", "uint16", "int8", "uint8"]
NP_OPS = {"eq": np.equal, "lt": np.less, "le": np.less_equal, "gt": np.greater, "ge": np.greater_equal}


@pytest.fixture(scope="module")
def gold():
    return np.load(GOLD)


def cases(gold, dtype):
    for op, n, incx, incy, inco, scal, start, size in gold[f"{dtype}_cmp_cases"]:
        yield int(op), int(n), int(incx), int(incy), int(inco), bool(scal), slice(int(start), int(start + size))


@pytest.mark.parametrize("dtype", DTYPES)
def test_oracle_matches_reference_goldens(O, gold, dtype):
    then, els = (1.5, -0.25) if dtype == "double" else (3, 5)
    checked = 0
    for op, n, incx, incy, inco, scal, sl in cases(gold, dtype):
        x, y = gold[f"{dtype}_cmp_x"][sl], gold[f"{dtype}_cmp_y"][sl]
        got = np.full(x.size, 7, x.dtype)
        O.cmp_typed_1d(dtype, O.CMP_OPS[op], n, x, incx, y[0].item() if scal else y, incy, got, inco, then, els)
        np.testing.assert_array_equal(got.view(np.uint8), gold[f"{dtype}_cmp_out"][sl].view(np.uint8),
                                      err_msg=f"{dtype} {O.CMP_OPS[op]} n={n} inc=({incx},{incy},{inco}) scal={scal}")
        checked += 1
    assert checked >= (100 if dtype == "double" else 40)


def test_fixture_pins_the_signed_blocks_of_uint32(gold):
    """At least one golden case separates the signed from the unsigned order:
    a :uint32 block element >= 2^31 against a small one."""
    seen = False
    for op, n, incx, incy, inco, scal, sl in cases(gold, "uint32"):
        if op == 0 or inco < 1 or n < 8 or scal:
            continue
        x = gold["uint32_cmp_x"][sl][: (n // 8) * 8].astype(np.int64)
        y = gold["uint32_cmp_y"][sl][: (n // 8) * 8].astype(np.int64)
        seen |= bool(np.any((x >= 2**31) != (y >= 2**31)))
    assert seen


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("scal", [False, True])
def test_closed_form(O, dtype, scal):
    npt = O.DTYPES[dtype][1]
    rng = np.random.default_rng(17)
    lanes = 32 // np.dtype(npt).itemsize
    for n, incx, incy, inco in [(3 * lanes + 5, 1, 1, 1), (2 * lanes + 1, 2, 3, 2), (lanes - 1, 1, 1, 1),
                                (2 * lanes, 1, 2, 0), (lanes + 3, 3, 1, -1)]:
        size = n * 3 + 1
        if dtype == "double":
            x = rng.integers(-2, 3, size).astype(npt)
            y = rng.integers(-2, 3, size).astype(npt)
            x[rng.random(size) < 0.1] = np.nan
            signed = np.float64
        else:
            info = np.iinfo(npt)
            x = rng.integers(info.min, info.max, size, endpoint=True).astype(npt)
            y = np.where(rng.random(size) < 0.3, x, rng.integers(info.min, info.max, size, endpoint=True)).astype(npt)
            signed = np.dtype(npt.__name__.lstrip("u"))
        ys = y[1].item()
        for op, fn in NP_OPS.items():
            got = np.full(size, 9, npt)
            offo = (n - 1) * -inco if inco < 0 else 0
            O.cmp_typed_1d(dtype, op, n, x, incx, ys if scal else y, incy, got, inco, 4, 6, offo=offo)
            xv = x[: n * incx: incx] if incx else x[:1].repeat(n)
            yv = np.full(n, ys, npt) if scal else y[: (n - 1) * incy + 1: incy]
            blocks = (n // lanes) * lanes if inco >= 1 else 0
            truth = fn(xv, yv)
            truth[:blocks] = fn(xv[:blocks].view(signed), yv[:blocks].view(signed))
            want = np.full(size, 9, npt)
            values = np.where(truth, 4, 6).astype(npt)
            if inco == 0:
                want[0] = values[-1]
            else:
                want[offo + np.arange(n) * inco] = values
            np.testing.assert_array_equal(got, want, err_msg=f"{dtype} {op} n={n} inc=({incx},{incy},{inco})")
