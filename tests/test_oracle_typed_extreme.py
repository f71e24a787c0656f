"""The oracle's restatement of waffe2_<prefix>{max,min} on :double and the integer
types against the golden vectors of the compiled reference
(tests/golden/typed_extreme_kernels.npz) and numpy's max / min.  Integer runs with a
non-unit increment that reach the 32-byte blocks are undefined in the reference
(strided lanes built by indexing a 4-lane vector, cl-waffe2-simd.c:54-107) and not in
the fixture; the extreme of a run of integers does not depend on the order anyway."""
import os

import numpy as np
import pytest

GOLD = os.path.join(os.path.dirname(__file__), "golden", "typed_extreme_kernels.npz")
DTYPES = ["double", "int32", "uint32", "int16", "uint16", "int8", "uint8"]


@pytest.mark.parametrize("dtype", DTYPES)
def test_oracle_matches_reference_goldens(O, dtype):
    gold = np.load(GOLD)
    rows = gold[f"{dtype}_extreme_cases"]
    assert len(rows) >= 4
    for k, (op, n, incx, start, size) in enumerate(rows):
        x = gold[f"{dtype}_extreme_x"][int(start):int(start + size)]
        got = O.extreme_typed_1d(dtype, ("max", "min")[int(op)], int(n), x, int(incx))
        assert got == gold[f"{dtype}_extreme_out"][k], (dtype, op, n, incx)


@pytest.mark.parametrize("dtype", DTYPES)
def test_oracle_is_the_extreme(O, dtype):
    npt = O.DTYPES[dtype][1]
    rng = np.random.default_rng(23)
    for n, incx, off in [(1, 1, 0), (7, 1, 3), (1000, 1, 0), (333, 3, 1), (64, 2, 0)]:
        size = n * incx + off + 1
        if dtype == "double":
            x = rng.standard_normal(size)
        else:
            info = np.iinfo(npt)
            x = rng.integers(info.min, info.max, size, endpoint=True).astype(npt)
        run = x[off: off + (n - 1) * incx + 1: incx]
        assert O.extreme_typed_1d(dtype, "max", n, x, incx, offx=off) == run.max()
        assert O.extreme_typed_1d(dtype, "min", n, x, incx, offx=off) == run.min()
