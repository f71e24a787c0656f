"""The oracle's restatement of waffe2_d{sin,...,pow} (SLEEF u10 on blocks of four, libm
on the remainder) against the golden vectors of the compiled reference
(tests/golden/double_unary_kernels.npz) -- bit for bit when SLEEF resolves, as both then
call the same routines -- and against numpy's binary64 functions within 1 ulp."""
import os

import numpy as np
import pytest

GOLD = os.path.join(os.path.dirname(__file__), "golden", "double_unary_kernels.npz")
NP = {"sin": np.sin, "cos": np.cos, "tanh": np.tanh, "log": np.log, "exp": np.exp, "sqrt": np.sqrt, "abs": np.abs,
      "tan": np.tan, "asin": np.arcsin, "acos": np.arccos, "atan": np.arctan, "sinh": np.sinh, "cosh": np.cosh,
      "log2": np.log2, "log10": np.log10, "log1p": np.log1p, "pow": lambda x: np.power(x, 2.5)}


def ulps(got, want):
    """Distance in units of the last place of `want` (binary64)."""
    return np.abs(got - want) / np.spacing(np.abs(want))


@pytest.mark.parametrize("op", list(NP))
def test_oracle_matches_reference_goldens(O, op):
    gold = np.load(GOLD)
    exact = O.sleef_available()
    for n, incx, inco, start, size in gold[f"{op}_cases"]:
        sl = slice(int(start), int(start + size))
        x = gold[f"{op}_x"][sl]
        got = np.full(x.size, 7.0)
        O.dunary_1d(op, int(n), x, int(incx), got, int(inco), p=2.5)
        want = gold[f"{op}_out"][sl]
        if exact:
            np.testing.assert_array_equal(got.view(np.uint64), want.view(np.uint64), err_msg=f"{op} n={n} inc=({incx},{inco})")
        else:
            assert np.max(ulps(got, want)) <= 1.0


@pytest.mark.parametrize("op", list(NP))
def test_oracle_is_the_function(O, op):
    rng = np.random.default_rng(3)
    if op in ("asin", "acos"):
        x = rng.uniform(-1, 1, 4001)
    elif op in ("log", "log2", "log10", "sqrt", "pow"):
        x = np.exp(rng.uniform(-5, 5, 4001))
    elif op == "log1p":
        x = np.expm1(rng.uniform(-5, 5, 4001))
    else:
        x = rng.uniform(-20, 20, 4001)
    got = np.zeros_like(x)
    O.dunary_1d(op, x.size, x, 1, got, 1, p=2.5)
    assert np.max(ulps(got, NP[op](x))) <= 2.0, op
