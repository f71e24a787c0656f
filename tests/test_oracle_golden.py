"""Pins the CPU oracle (oracle/waffe2_oracle.c) before anything trusts it:

* golden vectors produced by the reference's own compiled C kernels
  (tests/golden/simd_kernels.npz, written by tests/golden/make_golden.py);
* the compiled reference itself (oracle/_ref) on fresh random inputs where it
  is present;
* what the mathematics fixes: IEEE binary32 closed forms (numpy), float64
  truth within 1 ulp for the SLEEF u10 functions, exact special values;
* the reference's own test vectors (10 op 1 -> 11/9/10/10,
  base-impl/t/arithmetic.lisp:26-51; gemm vectors :120,135,142,148).
"""
import os

import numpy as np
import pytest

from helpers import assert_bit_equal, ulp_distance

GOLD = os.path.join(os.path.dirname(__file__), "golden", "simd_kernels.npz")
REGIMES = [(1, 1), (1, 0), (2, 1), (1, 3), (2, 2), (3, 0), (0, 1), (0, 0), (0, 2)]
SIZES = [1, 7, 8, 9, 31, 64, 67]


@pytest.fixture(scope="module")
def gold():
    return np.load(GOLD)


@pytest.mark.parametrize("op", ["add", "sub", "mul", "div"])
def test_binary_golden(O, gold, op):
    for n in SIZES:
        for incx, incy in REGIMES:
            key = f"bin_{op}_{n}_{incx}_{incy}"
            x = gold[key + "_x"].copy()
            O.binary_1d(op, n, x, incx, gold[key + "_y"].copy(), incy)
            assert_bit_equal(x, gold[key + "_out"], key)


@pytest.mark.parametrize("op,f", [("add", np.add), ("sub", np.subtract), ("mul", np.multiply),
                                  ("div", np.divide)])
def test_binary_closed_form(O, op, f):
    """IEEE binary32: one correctly rounded operation per element (numpy)."""
    rng = np.random.default_rng(1)
    x = rng.standard_normal(1001).astype(np.float32)
    y = rng.standard_normal(1001).astype(np.float32)
    got = x.copy()
    O.binary_1d(op, 1001, got, 1, y, 1)
    assert_bit_equal(got, f(x, y), op)
    got = x.copy()
    O.binary_1d(op, 500, got, 2, y, 0)  # strided x, scalar y
    want = x.copy()
    want[:1000:2] = f(x[:1000:2], y[0])
    assert_bit_equal(got, want, op + " strided/broadcast")
    # incx == 0: strictly sequential accumulation into x[0]
    got = x.copy()
    O.binary_1d(op, 100, got, 0, y, 1)
    acc = x[0]
    for i in range(100):
        acc = f(acc, y[i])
    assert got[0] == acc and np.array_equal(got[1:], x[1:])


def test_reference_tester_vectors(O):
    """add/sub/mul/div-tester: (100,100) of 10 op (100,100) of 1 -> 11/9/10/10;
    scalar testers likewise (base-impl/t/arithmetic.lisp:26-79)."""
    for op, want in [("add", 11.0), ("sub", 9.0), ("mul", 10.0), ("div", 10.0)]:
        x = np.full(10000, 10.0, np.float32)
        O.binary_1d(op, 10000, x, 1, np.ones(10000, np.float32), 1)
        assert np.all(x == want)
        x = np.full(10000, 10.0, np.float32)
        O.binary_1d(op, 10000, x, 1, np.ones(1, np.float32), 0)
        assert np.all(x == want)


@pytest.mark.skipif(not os.path.exists(os.path.join(os.path.dirname(__file__), "..", "oracle", "_ref",
                                                    "libwaffe2_simd_ref.so")),
                    reason="oracle/_ref not built (needs the reference checkout)")
def test_oracle_equals_compiled_reference(O):
    if O.ref() is None:
        pytest.skip("oracle/_ref does not load here")
    rng = np.random.default_rng(7)
    for op in ("add", "sub", "mul", "div"):
        for n in (5, 8, 100, 1003):
            for incx, incy in REGIMES:
                x = rng.standard_normal(3100).astype(np.float32)
                y = rng.uniform(0.5, 1.5, 3100).astype(np.float32)
                a, b = x.copy(), x.copy()
                O.binary_1d(op, n, a, incx, y, incy)
                O.binary_1d(op, n, b, incx, y, incy, use_ref=True)
                assert_bit_equal(a, b, f"{op} {n} {incx} {incy}")
    for op, lo, hi in [("exp", -10, 10), ("tanh", -10, 10), ("sin", -100, 100), ("log", 1e-3, 1e3),
                       ("sqrt", 0, 100), ("cos", -100, 100), ("abs", -1, 1)]:
        for n, incx, inco in [(1003, 1, 1), (500, 2, 1), (500, 1, 2), (77, 0, 1)]:
            x = rng.uniform(lo, hi, 1100).astype(np.float32)
            a = np.zeros(1100, np.float32)
            b = np.zeros(1100, np.float32)
            O.unary_1d(op, n, x, incx, a, inco)
            O.unary_1d(op, n, x, incx, b, inco, use_ref=True)
            assert_bit_equal(a, b, f"{op} {n} {incx} {inco}")


UNARY = ["exp", "tanh", "sin", "cos", "log", "sqrt", "abs"]


@pytest.mark.parametrize("op", UNARY)
def test_unary_golden(O, gold, op):
    if not O.sleef_available():
        pytest.skip("no SLEEF provider: the oracle runs on libm and is only within 1 ulp of the goldens")
    x = gold[f"un_{op}_range_x"]
    got = np.zeros_like(x)
    O.unary_1d(op, x.size, x, 1, got, 1)
    assert_bit_equal(got, gold[f"un_{op}_range_out"], op)
    got = np.zeros(gold["edge_x"].size, np.float32)
    with np.errstate(all="ignore"):
        O.unary_1d(op, got.size, gold["edge_x"], 1, got, 1)
    assert_bit_equal(got, gold[f"un_{op}_edge_out"], op + " edge")
    for n, incx, inco in [(13, 2, 1), (16, 1, 3), (9, 0, 1)]:
        got = np.full(64, 7.0, np.float32)
        O.unary_1d(op, n, x, incx, got, inco)
        assert_bit_equal(got, gold[f"un_{op}_{n}_{incx}_{inco}_out"], f"{op} {n} {incx} {inco}")


@pytest.mark.parametrize("op", UNARY)
def test_unary_against_float64_truth(O, gold, op):
    """SLEEF u10 promises <= 1.0 ulp (sqrt u05: correctly rounded); the goldens
    and the oracle must honour it against numpy float64."""
    x = gold[f"un_{op}_range_x"]
    truth = getattr(np, "abs" if op == "abs" else op)(x.astype(np.float64)).astype(np.float32)
    limit = 0 if op in ("sqrt", "abs") else 1
    assert ulp_distance(gold[f"un_{op}_range_out"], truth).max() <= limit
    got = np.zeros_like(x)
    O.unary_1d(op, x.size, x, 1, got, 1)
    assert ulp_distance(got, truth).max() <= limit


MORE_GOLD = os.path.join(os.path.dirname(__file__), "golden", "unary_more_kernels.npz")
MORE = ["tan", "asin", "acos", "atan", "sinh", "cosh", "log2", "log10", "log1p"]
MORE_TRUTH = {"tan": np.tan, "asin": np.arcsin, "acos": np.arccos, "atan": np.arctan, "sinh": np.sinh,
              "cosh": np.cosh, "log2": np.log2, "log10": np.log10, "log1p": np.log1p}


@pytest.mark.parametrize("op", MORE)
def test_more_unary_golden_and_truth(O, op):
    """Tan, ASin, ACos, ATan, SinH, CosH, Log2, Log10, Log1p
    (cl-waffe2-simd.c:650-694): the oracle reproduces the compiled reference bit
    for bit (same SLEEF symbols, same block/tail structure) and both are within
    1 ulp of float64."""
    gold = np.load(MORE_GOLD)
    x = gold[f"un_{op}_range_x"]
    truth = MORE_TRUTH[op](x.astype(np.float64)).astype(np.float32)
    assert ulp_distance(gold[f"un_{op}_range_out"], truth).max() <= 1
    if not O.sleef_available():
        pytest.skip("no SLEEF provider")
    got = np.zeros_like(x)
    O.unary_1d(op, x.size, x, 1, got, 1)
    assert_bit_equal(got, gold[f"un_{op}_range_out"], op)
    got = np.zeros(gold["edge_x"].size, np.float32)
    with np.errstate(all="ignore"):
        O.unary_1d(op, got.size, gold["edge_x"], 1, got, 1)
    assert_bit_equal(got, gold[f"un_{op}_edge_out"], op + " edge")
    for n, incx, inco in [(13, 2, 1), (16, 1, 3), (9, 0, 1)]:
        got = np.full(64, 7.0, np.float32)
        O.unary_1d(op, n, x, incx, got, inco)
        assert_bit_equal(got, gold[f"un_{op}_{n}_{incx}_{inco}_out"], f"{op} {n} {incx} {inco}")


def test_unary_special_values(O):
    def f(op, v):
        out = np.zeros(1, np.float32)
        with np.errstate(all="ignore"):
            O.unary_1d(op, 1, np.array([v], np.float32), 1, out, 1)
        return out[0]
    assert f("exp", 0.0) == 1.0 and f("log", 1.0) == 0.0 and f("sin", 0.0) == 0.0
    assert f("tanh", np.inf) == 1.0 and f("tanh", -np.inf) == -1.0 and f("cos", 0.0) == 1.0
    assert f("log", 0.0) == -np.inf and np.isnan(f("log", -1.0)) and f("exp", -np.inf) == 0.0
    assert f("sqrt", 4.0) == 2.0 and f("abs", -3.5) == 3.5


def test_pow_and_maxmin_golden(O, gold):
    for p in (2.0, 3.0, 0.5, 2.5, -1.0):
        x = gold[f"pow_{p}_x"]
        got = np.zeros_like(x)
        O.pow_1d(x.size, x, 1, p, got, 1)
        if O.sleef_available():
            assert_bit_equal(got, gold[f"pow_{p}_out"], f"pow {p}")
        with np.errstate(all="ignore"):
            truth = np.power(x.astype(np.float64), p).astype(np.float32)
        assert ulp_distance(gold[f"pow_{p}_out"], truth).max() <= 1
    for n, inc in [(1, 1), (5, 1), (8, 1), (67, 1), (40, 3)]:
        x = gold[f"max_{n}_{inc}_x"]
        assert O.maxmin_1d("max", n, x, inc) == gold[f"max_{n}_{inc}_out"] == x[::inc][:n].max()
        assert O.maxmin_1d("min", n, x, inc) == gold[f"min_{n}_{inc}_out"] == x[::inc][:n].min()


def test_copy(O):
    y = np.arange(40, dtype=np.float32)
    x = np.zeros(40, np.float32)
    O.copy_1d(10, y, 3, x, 2)
    assert x[:20:2].tolist() == y[:30:3].tolist() and np.all(x[1::2] == 0)


def test_gemm_reference_vectors(O):
    """matmul-tester vectors (base-impl/t/arithmetic.lisp:120,135,142,148) and
    the column == row-major equivalence (backends/cpu/t/arithmetic.lisp:53-68)."""
    a33 = np.arange(9, dtype=np.float32).reshape(3, 3)
    a34 = np.arange(12, dtype=np.float32).reshape(3, 4)
    assert O.matmul_rowmajor(a33, a33).ravel().tolist() == [15, 18, 21, 42, 54, 66, 69, 90, 111]
    assert O.matmul_rowmajor(a34, a34, trans_b=True).ravel().tolist() == [14, 38, 62, 38, 126, 214, 62, 214, 366]
    assert O.matmul_rowmajor(a34, a34, trans_a=True).ravel().tolist() == [
        80, 92, 104, 116, 92, 107, 122, 137, 104, 122, 140, 158, 116, 137, 158, 179]
    assert O.matmul_rowmajor(a33, a33, trans_a=True, trans_b=True).ravel().tolist() == [
        15, 42, 69, 18, 54, 90, 21, 66, 111]


def test_gemm_against_float64(O):
    rng = np.random.default_rng(3)
    for ta in ("N", "T"):
        for tb in ("N", "T"):
            m, n, k = 13, 9, 21
            A = rng.standard_normal((k, m) if ta == "N" else (m, k)).astype(np.float32)  # column-major storage
            B = rng.standard_normal((n, k) if tb == "N" else (k, n)).astype(np.float32)
            Cm = rng.standard_normal((n, m)).astype(np.float32)
            opA = A.T if ta == "N" else A          # (m, k)
            opB = B.T if tb == "N" else B          # (k, n)
            want = 0.5 * (opA.astype(np.float64) @ opB.astype(np.float64)) + 2.0 * Cm.T.astype(np.float64)
            got = Cm.copy().ravel()
            O.sgemm(ta, tb, m, n, k, 0.5, A.ravel(), A.shape[1], B.ravel(), B.shape[1], 2.0, got, m)
            np.testing.assert_allclose(got.reshape(n, m).T, want, rtol=1e-5, atol=1e-5)


# ---------------------------------------------------------------------------
# compare / where (cl-waffe2-simd.c:385-513)
# ---------------------------------------------------------------------------
CMP_GOLD = os.path.join(os.path.dirname(__file__), "golden", "compare_kernels.npz")
CMP_REGIMES = [(1, 1, 1), (1, 0, 1), (2, 1, 1), (1, 3, 2), (2, 2, 3), (0, 1, 1), (1, 1, 0), (3, 0, 0)]
CMP_NUMPY = {"eq": np.equal, "lt": np.less, "le": np.less_equal, "gt": np.greater, "ge": np.greater_equal}


@pytest.fixture(scope="module")
def cmp_gold():
    return np.load(CMP_GOLD)


@pytest.mark.parametrize("op", ["eq", "lt", "le", "gt", "ge"])
def test_compare_golden(O, cmp_gold, op):
    """Tensor and scalar right-hand sides, every stride regime (a stride-0 `out`
    keeps the last element's result), bitwise against the compiled reference's
    outputs."""
    for n in (1, 7, 8, 9, 31, 67):
        for incx, incy, inco in CMP_REGIMES:
            key = f"cmp_{op}_{n}_{incx}_{incy}_{inco}"
            x, y = cmp_gold[key + "_x"], cmp_gold[key + "_y"]
            got = np.full(x.size, 9.0, np.float32)
            O.cmp_1d(op, n, x, incx, y, incy, got, inco, 2.5, -1.5)
            assert_bit_equal(got, cmp_gold[key + "_out"], key)
            got = np.full(x.size, 9.0, np.float32)
            O.cmp_scal_1d(op, n, x, incx, got, inco, 1.0, 2.5, -1.5)
            assert_bit_equal(got, cmp_gold[key + "_scal_out"], key + " scal")
            # what the definition fixes, where `out` is not collapsed
            if inco >= 1:
                xs = x[::incx][:n] if incx else np.repeat(x[0], n)
                ys = y[::incy][:n] if incy else np.repeat(y[0], n)
                want = np.where(CMP_NUMPY[op](xs, ys), np.float32(2.5), np.float32(-1.5))
                assert_bit_equal(cmp_gold[key + "_out"][::inco][:n], want, key + " numpy")


@pytest.mark.parametrize("op", ["eq", "lt", "le", "gt", "ge"])
def test_compare_special_values(O, cmp_gold, op):
    """NaN compares false under every predicate, -0 == +0, infinities order."""
    edge = cmp_gold["cmp_edge"]
    xs, ys = np.repeat(edge, edge.size), np.tile(edge, edge.size)
    got = np.zeros(xs.size, np.float32)
    O.cmp_1d(op, xs.size, xs, 1, ys, 1, got, 1, 1.0, 0.0)
    assert_bit_equal(got, cmp_gold[f"cmp_{op}_edge_out"], op)
    with np.errstate(invalid="ignore"):
        assert_bit_equal(got, CMP_NUMPY[op](xs, ys).astype(np.float32), op + " numpy")
    nan_rows = np.isnan(xs) | np.isnan(ys)
    assert not got[nan_rows].any()


def test_index_of_extreme_value(O):
    """orc_ismax / orc_ismin restate OpenBLAS' ismax_ / ismin_ (1-based, first
    occurrence).  Pinned by the definition on tie-rich data and strides."""
    rng = np.random.default_rng(12)
    for n, inc in [(1, 1), (2, 1), (9, 1), (64, 1), (100, 3), (1000, 2)]:
        x = rng.integers(-4, 5, n * inc + 1).astype(np.float32)
        run = x[::inc][:n]
        assert O.argmaxmin_1d("max", n, x, inc) == int(np.argmax(run))
        assert O.argmaxmin_1d("min", n, x, inc) == int(np.argmin(run))
        assert run[O.argmaxmin_1d("max", n, x, inc)] == O.maxmin_1d("max", n, x, inc)
    x = np.array([1, 5, 5, 0, 0, 5], np.float32)
    assert O.argmaxmin_1d("max", 6, x, 1) == 1 and O.argmaxmin_1d("min", 6, x, 1) == 3


def test_inv(O):
    """x <- 1 / x (cl-waffe2-simd.c:290-302): equals the IEEE binary32 division,
    equals the compiled reference where present, and a stride-0 run is inverted
    n times."""
    rng = np.random.default_rng(4)
    x = np.concatenate([rng.standard_normal(1000), [0.0, -0.0, np.inf, 1e-45, 3e38, 1.0, 3.0]]).astype(np.float32)
    for inc in (1, 2, 3):
        n = x.size // inc
        got = x.copy()
        with np.errstate(all="ignore"):
            O.inv_1d(n, got, inc)
            want = x.copy()
            want[:n * inc:inc] = np.float32(1.0) / x[:n * inc:inc]
        assert_bit_equal(got, want, f"inv inc={inc}")
        if O.ref() is not None:
            r = x.copy()
            with np.errstate(all="ignore"):
                O.inv_1d(n, r, inc, use_ref=True)
            assert_bit_equal(got, r, "inv vs reference")
    one = np.array([3.0], np.float32)
    O.inv_1d(5, one, 0)
    want = np.float32(3.0)
    for _ in range(5):
        want = np.float32(1.0) / want
    assert one[0] == want


def test_im2col_golden(O):
    """orc_im2col / orc_col2im against the outputs of the reference's im2col.c
    (compiled into oracle/_ref) on the geometries `unfold` produces, bitwise;
    elements the reference's walk does not reach keep their previous value;
    with no padding and stride 1 the result is the textbook unfold."""
    import importlib.util
    spec = importlib.util.spec_from_file_location(
        "make_golden", os.path.join(os.path.dirname(__file__), "golden", "make_golden.py"))
    mg = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mg)
    gold = np.load(os.path.join(os.path.dirname(__file__), "golden", "im2col_kernels.npz"))
    for idx, case in enumerate(mg.IM2COL_CASES):
        N, Cc, H, W, Ho, Wo, kh, kw = mg.im2col_geometry(case)
        _, _, _, _, k, s, p = case
        im = gold[f"im2col_{idx}_im"]
        col = np.full((N, Cc, kh, kw, Ho, Wo), 7.0, np.float32)
        O.im2col(col, im, N, Cc, H, W, Ho, Wo, kh, kw, p, s, (1, 1))
        assert_bit_equal(col, gold[f"im2col_{idx}_col"], f"im2col case {idx}")
        back = np.full(im.shape, 5.0, np.float32)
        O.col2im(gold[f"col2im_{idx}_col"], back, N, Cc, H, W, Ho, Wo, kh, kw, p, s, (1, 1))
        assert_bit_equal(back, gold[f"col2im_{idx}_im"], f"col2im case {idx}")
        if O.im2col_ref_available():
            col2 = np.full(col.shape, 7.0, np.float32)
            O.im2col(col2, im, N, Cc, H, W, Ho, Wo, kh, kw, p, s, (1, 1), use_ref=True)
            assert_bit_equal(col, col2, "oracle vs compiled reference")
    # closed form: case 0 (5x5, 3x3, stride 1, no padding) is the sliding window
    im = gold["im2col_0_im"][0, 0]
    want = np.lib.stride_tricks.sliding_window_view(im, (3, 3)).transpose(2, 3, 0, 1)
    assert_bit_equal(gold["im2col_0_col"][0, 0], np.ascontiguousarray(want), "sliding window")


def test_lisp_loop_nodes_follow_their_definitions(O):
    """SignNode, SquareNode, ASinHNode, ACosHNode, ATanHNode (LispTensor's per-element
    loop in the reference; no SIMD kernel, no golden vectors): the oracle against the
    float64 closed forms, strided and with special values."""
    rng = np.random.default_rng(5)
    truth = {"sign": np.sign, "square": np.square, "asinh": np.arcsinh, "acosh": np.arccosh, "atanh": np.arctanh}
    ranges = {"sign": (-3, 3), "square": (-100, 100), "asinh": (-1e4, 1e4), "acosh": (1, 1e4), "atanh": (-0.999, 0.999)}
    for op in O.LISP_UNARY_NAMES:
        lo, hi = ranges[op]
        for n, incx, inco in [(1000, 1, 1), (333, 3, 2), (7, 1, 5)]:
            x = rng.uniform(lo, hi, n * incx).astype(np.float32)
            out = np.full(n * inco, 99.0, np.float32)
            O.unary_1d(op, n, x, incx, out, inco)
            with np.errstate(all="ignore"):
                want = truth[op](x[::incx][:n].astype(np.float64)).astype(np.float32)
            assert np.array_equal(out[::inco][:n], want) or \
                np.abs(out[::inco][:n].view(np.int32).astype(np.int64) - want.view(np.int32)).max() <= 1, op
            if inco > 1:
                assert np.all(out.reshape(-1, inco)[:, 1:] == 99.0)
    edge = np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 1.0, -1.0, 0.5], np.float32)
    out = np.zeros_like(edge)
    O.unary_1d("sign", edge.size, edge, 1, out, 1)
    assert out[:4].tolist() == [0.0, -0.0, 1.0, -1.0] and np.signbit(out[1]) and np.isnan(out[4])
    O.unary_1d("atanh", edge.size, edge, 1, out, 1)
    assert out[5] == np.inf and out[6] == -np.inf and np.isnan(out[2]) and out[0] == 0.0
    O.unary_1d("acosh", edge.size, edge, 1, out, 1)
    assert out[5] == 0.0 and np.isnan(out[7]) and out[2] == np.inf


def test_gpt2_positional_embedding_restatement(O):
    """The restated loop of examples/gpt-2/utils.lisp:19-66 equals the closed form the node documents,
    add(WTE[CTX], WPE[position]), exactly; ids round half to even as (round x) does."""
    rng = np.random.default_rng(3)
    wte = rng.standard_normal((40, 10)).astype(np.float32)
    wpe = rng.standard_normal((12, 10)).astype(np.float32)
    ctx = rng.integers(0, 40, (3, 9)).astype(np.float32)
    got = O.gpt2_positional_embedding(ctx, wte, wpe)
    want = wte[ctx.astype(int)] + wpe[np.arange(9)][None]
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    halves = O.gpt2_positional_embedding(np.array([[0.5, 1.5, 2.5]], np.float32), wte, np.zeros_like(wpe))
    assert np.array_equal(halves[0], wte[[0, 2, 2]])
