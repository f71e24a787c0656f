"""GPU parity of the unary math kernels on :double tensors: within 2 ulp (binary64) of
the golden vectors of the compiled reference (SLEEF u10 / libm) and of the oracle at
larger sizes, special values, the node layer on views."""
import ctypes as C
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

GOLD = os.path.join(os.path.dirname(__file__), "golden", "double_unary_kernels.npz")
OPS = ["sin", "cos", "tanh", "log", "exp", "sqrt", "abs", "tan", "asin", "acos", "atan", "sinh", "cosh", "log2",
       "log10", "log1p", "pow"]
TOL_ULP = 2.0


def ulps(got, want):
    with np.errstate(invalid="ignore"):
        d = np.abs(got - want) / np.spacing(np.abs(want))
    same = (got == want) | (np.isnan(got) & np.isnan(want))
    return np.where(same, 0.0, d)


def run_1d(W, op, n, x, incx, inco, size, p=2.5, fill=7.0):
    lib = W.lib.get()
    dx = W.HIPTensor.from_numpy(x, dtype="double")
    dout = W.HIPTensor.from_numpy(np.full(size, fill), dtype="double")
    if op == "pow":
        W.lib.check(lib.wf2hip_dpow(n, C.c_void_p(dx.ptr), incx, p, C.c_void_p(dout.ptr), inco))
    else:
        W.lib.check(getattr(lib, f"wf2hip_d{op}")(n, C.c_void_p(dx.ptr), incx, C.c_void_p(dout.ptr), inco))
    return dout.numpy()


@pytest.mark.parametrize("op", OPS)
def test_against_reference_goldens(gpu, op):
    gold = np.load(GOLD)
    worst = 0.0
    for n, incx, inco, start, size in gold[f"{op}_cases"]:
        sl = slice(int(start), int(start + size))
        x, want = gold[f"{op}_x"][sl], gold[f"{op}_out"][sl]
        got = run_1d(gpu, op, int(n), x, int(incx), int(inco), x.size)
        u = ulps(got, want)
        worst = max(worst, float(u.max()))
        assert u.max() <= TOL_ULP, f"{op} n={n} inc=({incx},{inco}): {u.max()} ulp"
        untouched = want == 7.0
        np.testing.assert_array_equal(got[untouched], want[untouched])


@pytest.mark.parametrize("op", OPS)
def test_against_oracle_at_size(gpu, O, op):
    rng = np.random.default_rng(59)
    n = 200003
    if op in ("asin", "acos"):
        x = rng.uniform(-1, 1, n)
    elif op in ("log", "log2", "log10", "sqrt"):
        x = np.exp(rng.uniform(-300, 300, n))
    elif op == "log1p":
        x = np.expm1(rng.uniform(-30, 30, n))
    elif op in ("exp", "sinh", "cosh"):
        x = rng.uniform(-700, 700, n)
    elif op in ("sin", "cos", "tan"):
        x = rng.uniform(-1, 1, n) * 10.0 ** rng.integers(-6, 9, n)
    elif op == "pow":
        x = np.exp(rng.uniform(-20, 20, n))
    else:
        x = rng.uniform(-30, 30, n)
    want = np.zeros(n)
    O.dunary_1d(op, n, x, 1, want, 1, p=2.5)
    got = run_1d(gpu, op, n, x, 1, 1, n)
    u = ulps(got, want)
    assert u.max() <= TOL_ULP, f"{op}: {u.max()} ulp at x = {x[int(u.argmax())]!r}"
    # unaligned start and the odd remainder
    got = np.full(1001, 7.0)
    dx = gpu.HIPTensor.from_numpy(x[:1001].copy(), dtype="double")
    dout = gpu.HIPTensor.from_numpy(got, dtype="double")
    lib = gpu.lib.get()
    if op == "pow":
        gpu.lib.check(lib.wf2hip_dpow(999, C.c_void_p(dx.ptr + 8), 1, 2.5, C.c_void_p(dout.ptr + 8), 1))
    else:
        gpu.lib.check(getattr(lib, f"wf2hip_d{op}")(999, C.c_void_p(dx.ptr + 8), 1, C.c_void_p(dout.ptr + 8), 1))
    res = dout.numpy()
    assert ulps(res[1:1000], want[1:1000]).max() <= TOL_ULP and res[0] == 7.0 and res[1000] == 7.0


def test_special_values(gpu):
    inf, nan = np.inf, np.nan
    x = np.array([0.0, -0.0, inf, -inf, nan, 1.0, -1.0, 2.0, 710.0, -746.0, 5e-324, 1e308])
    with np.errstate(all="ignore"):
        table = {"exp": np.exp(x), "log": np.log(x), "sqrt": np.sqrt(x), "abs": np.abs(x), "tanh": np.tanh(x),
                 "sin": np.sin(x), "cos": np.cos(x), "atan": np.arctan(x), "log1p": np.log1p(x),
                 "asin": np.arcsin(x), "sinh": np.sinh(x), "cosh": np.cosh(x)}
    for op, want in table.items():
        got = run_1d(gpu, op, x.size, x, 1, 1, x.size)
        assert ulps(got, want).max() <= TOL_ULP, (op, got, want)
        np.testing.assert_array_equal(np.isnan(got), np.isnan(want), err_msg=op)
        zero = want == 0
        np.testing.assert_array_equal(np.signbit(got[zero]), np.signbit(want[zero]), err_msg=op)


def test_nodes_on_views(gpu):
    W = gpu
    F = W.functional
    rng = np.random.default_rng(61)
    A = rng.uniform(0.1, 4.0, (6, 40, 34))
    dA = F.from_numpy(A, dtype="double")
    for fn, ref in ((F.exp, np.exp), (F.loge, np.log), (F.tanh, np.tanh), (F.sin, np.sin), (F.sqrt, np.sqrt)):
        got = fn(dA)
        assert got.dtype == "double"
        assert ulps(got.numpy(), ref(A)).max() <= TOL_ULP
        v = dA.view((1, 5), (0, 40, 3), (1, 33, 2))
        assert ulps(fn(v).numpy(), ref(A[1:5, 0:40:3, 1:33:2][:, :13])).max() <= TOL_ULP
        p = dA.permute(2, 0, 1)
        assert ulps(fn(p).numpy(), ref(np.transpose(A, (2, 0, 1)))).max() <= TOL_ULP
    assert ulps(F.expt(dA, 1.75).numpy(), A ** 1.75).max() <= TOL_ULP
    with pytest.raises(W.nodes.NodeNotFound):
        F.exp(F.from_numpy(np.ones((2, 2), np.int32), dtype="int32"))
