"""GPU parity of MatMulNode on :double tensors (wf2hip_dgemm*).

The CPU backend sends these products to BLAS dgemm_
(source/backends/cpu/matrix-ops.lisp:12-112, blas-functions.lisp:34-38), a
dependency that is not part of the reference's sources.  What the mathematics
fixes is used instead: the product evaluated in extended precision
(np.longdouble) bounds the error of any binary64 evaluation order by
k * 2^-53 * |A| |B|; numpy's own dgemm is checked beside it.  Bar: error
<= 4 * k * 2^-53 relative to |A| |B| (far below the 1e-5 of the float path).
"""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

EPS = 2.0 ** -53


def D(array):
    """A :double device tensor holding ``array``."""
    import importlib

    return importlib.import_module("cl-waffe2_amd").HIPTensor.from_numpy(array, dtype="double")


def _check(got, opA, opB, extra=None, what=""):
    k = opA.shape[1]
    want = opA.astype(np.longdouble) @ opB.astype(np.longdouble)
    scale = np.abs(opA) @ np.abs(opB)
    if extra is not None:
        want = want + extra.astype(np.longdouble)
        scale = scale + np.abs(extra)
    err = np.max(np.abs(got.astype(np.longdouble) - want) / np.maximum(scale, 1e-300))
    assert err <= 4 * max(k, 1) * EPS, f"{what}: relative error {float(err):.3e}"


@pytest.mark.parametrize("m,n,k", [(1, 1, 1), (3, 5, 7), (64, 64, 16), (65, 63, 17), (130, 257, 300), (256, 192, 1024)])
@pytest.mark.parametrize("ta", [False, True])
@pytest.mark.parametrize("tb", [False, True])
def test_double_matmul_random(gpu, m, n, k, ta, tb):
    """Every transpose form, sizes on and off the 64 x 64 x 16 tile."""
    F = gpu.functional
    rng = np.random.default_rng(m * 1000 + n * 10 + k)
    A = rng.standard_normal((k, m) if ta else (m, k))
    B = rng.standard_normal((n, k) if tb else (k, n))
    a, b = F.from_numpy(A, dtype="double"), F.from_numpy(B, dtype="double")
    assert a.dtype == "double"
    out = F.matmul(F.t(a) if ta else a, F.t(b) if tb else b)
    assert out.dtype == "double" and out.shape == [m, n]
    opA, opB = (A.T if ta else A), (B.T if tb else B)
    _check(out.numpy(), opA, opB, what=f"{m}x{n}x{k} {ta} {tb}")
    # numpy's dgemm agrees to the same bound
    np.testing.assert_allclose(out.numpy(), opA @ opB, rtol=0, atol=8 * k * EPS * float(np.max(np.abs(opA) @ np.abs(opB))))


def test_double_matmul_keeps_what_float_loses(gpu):
    """A product whose binary32 evaluation is visibly wrong: (1 + 2^-30)^2
    summed with -1 needs more than 24 bits."""
    F = gpu.functional
    x = 1.0 + 2.0 ** -30
    A = np.array([[x, 1.0]], dtype=np.float64)
    B = np.array([[x], [-1.0]], dtype=np.float64)
    got = F.matmul(D(A), D(B)).numpy()
    assert got[0, 0] == x * x - 1.0 != 0.0


def test_double_matmul_batched_and_broadcast(gpu):
    """Batch axes, a rank-2 weight against a rank-3 activation, transposed heads."""
    F = gpu.functional
    rng = np.random.default_rng(5)
    X = rng.standard_normal((4, 50, 24))
    Wt = rng.standard_normal((24, 36))
    got = F.matmul(D(X), D(Wt)).numpy()
    for b in range(4):
        _check(got[b], X[b], Wt, what=f"batch {b}")
    Q = rng.standard_normal((2, 3, 40, 16))
    K = rng.standard_normal((2, 3, 40, 16))
    got = F.matmul(D(Q), F.t(D(K))).numpy()
    assert got.shape == (2, 3, 40, 40)
    for b in range(2):
        for h in range(3):
            _check(got[b, h], Q[b, h], K[b, h].T, what=f"head {b},{h}")


def test_dgemm_column_major_contract(gpu):
    """wf2hip_dgemm keeps Fortran dgemm_ semantics: column-major storage, leading
    dimensions larger than the matrices, alpha and beta, padding rows untouched,
    beta = 0 never reads C, bad arguments are refused."""
    W = gpu
    lib = W.lib.get()
    rng = np.random.default_rng(77)
    dp = lambda t: C.c_void_p(t.ptr)
    for ca in "NT":
        for cb in "NC":
            m, n, k = 37, 29, 53
            lda = (m if ca == "N" else k) + 3
            ldb = (k if cb == "N" else n) + 2
            ldc = m + 4
            A = rng.standard_normal(lda * (k if ca == "N" else m))
            B = rng.standard_normal(ldb * (n if cb == "N" else k))
            Cm = rng.standard_normal(ldc * n)
            A2, B2, C2 = A.reshape(-1, lda).T, B.reshape(-1, ldb).T, Cm.reshape(-1, ldc).T
            opA = A2[:m, :k] if ca == "N" else A2[:k, :m].T
            opB = B2[:k, :n] if cb == "N" else B2[:n, :k].T
            dA, dB, dC = D(A), D(B), D(Cm)
            W.lib.check(lib.wf2hip_dgemm(ca.encode(), cb.encode(), m, n, k, 0.5, dp(dA), lda, dp(dB), ldb, -2.0,
                                         dp(dC), ldc))
            got = dC.numpy().reshape(-1, ldc).T
            _check(got[:m, :n], 0.5 * opA, opB, extra=-2.0 * C2[:m, :n], what=f"{ca}{cb}")
            np.testing.assert_array_equal(got[m:, :], C2[m:, :])
    eye = D(np.eye(4).ravel())
    nanC = D(np.full(16, np.nan))
    W.lib.check(lib.wf2hip_dgemm(b"N", b"N", 4, 4, 4, 1.0, dp(eye), 4, dp(eye), 4, 0.0, dp(nanC), 4))
    np.testing.assert_array_equal(nanC.numpy().reshape(4, 4), np.eye(4))
    assert lib.wf2hip_dgemm(b"X", b"N", 4, 4, 4, 1.0, dp(eye), 4, dp(eye), 4, 0.0, dp(nanC), 4) == -1
    assert lib.wf2hip_dgemm(b"N", b"N", 4, 4, 4, 1.0, dp(eye), 2, dp(eye), 4, 0.0, dp(nanC), 4) == -1
    # k = 0: C <- beta C
    c = D(np.arange(16, dtype=np.float64))
    W.lib.check(lib.wf2hip_dgemm(b"N", b"N", 4, 4, 0, 1.0, dp(eye), 4, dp(eye), 1, 3.0, dp(c), 4))
    np.testing.assert_array_equal(c.numpy(), 3.0 * np.arange(16))


def test_double_matmul_rejects_mixed_dtypes_and_fused_epilogues(gpu):
    F = gpu.functional
    a = D(np.ones((4, 4)))
    b = F.from_numpy(np.ones((4, 4), dtype=np.float32))
    with pytest.raises(ValueError):
        F.matmul(a, b)
    with pytest.raises(ValueError):
        F.matmul(a, a, activation="gelu")


@pytest.mark.parametrize("ta", [False, True])
@pytest.mark.parametrize("tb", [False, True])
def test_double_matmul_large_tiles(gpu, ta, tb):
    """Enough 128 x 128 tiles to fill the chip twice over select the large-tile
    form of the kernel; sizes off the tile in every dimension."""
    F = gpu.functional
    batch, m, n, k = 26, 500, 515, 70
    rng = np.random.default_rng(11 + 2 * ta + tb)
    A = rng.standard_normal((batch, k, m) if ta else (batch, m, k))
    B = rng.standard_normal((batch, n, k) if tb else (batch, k, n))
    a, b = D(A), D(B)
    got = F.matmul(F.t(a) if ta else a, F.t(b) if tb else b).numpy()
    assert got.shape == (batch, m, n)
    opA = A.transpose(0, 2, 1) if ta else A
    opB = B.transpose(0, 2, 1) if tb else B
    want = opA @ opB
    scale = np.abs(opA) @ np.abs(opB)
    assert np.max(np.abs(got - want) / scale) <= 8 * k * EPS
    _check(got[0], opA[0], opB[0], what="first matrix, extended precision")
    _check(got[-1], opA[-1], opB[-1], what="last matrix, extended precision")


@pytest.mark.parametrize("m,n,k", [(10, 10, 1 << 17), (64, 64, 40000), (3, 200, 2048), (130, 70, 5003)])
@pytest.mark.parametrize("ta", [False, True])
@pytest.mark.parametrize("tb", [False, True])
def test_double_matmul_few_outputs_long_k(gpu, m, n, k, ta, tb):
    """Few output tiles over a long K run as slices of K folded afterwards: K on and off the slice length,
    every transpose form, and alpha, beta and a padded ldc through the C-ABI."""
    W = gpu
    F = W.functional
    rng = np.random.default_rng(m + n + k)
    A = rng.standard_normal((k, m) if ta else (m, k))
    B = rng.standard_normal((n, k) if tb else (k, n))
    a, b = D(A), D(B)
    out = F.matmul(F.t(a) if ta else a, F.t(b) if tb else b)
    opA, opB = (A.T if ta else A), (B.T if tb else B)
    _check(out.numpy(), opA, opB, what=f"{m}x{n}x{k} {ta} {tb}")
    # column-major call: C (m x n, ldc = m + 3) <- 0.5 op(A) op(B) - 2 C; the row-major arrays above are the
    # column-major transposes, so op(A) here is opB^T ... use the Fortran reading directly instead
    lib = W.lib.get()
    dp = lambda t: C.c_void_p(t.ptr)
    ldc = m + 3
    Cm = rng.standard_normal(ldc * n)
    dC = D(Cm)
    # A as stored is (k, m) row-major when ta, i.e. column-major m x k with lda = m: op = 'N'
    Acm = np.ascontiguousarray(opA.T) if not ta else np.ascontiguousarray(opA)   # column-major m x k / k x m
    Bcm = np.ascontiguousarray(opB.T) if not tb else np.ascontiguousarray(opB)
    dA, dB = D(Acm.ravel()), D(Bcm.ravel())
    # Acm (not ta): array (k, m) row-major = column-major m x k, lda = m, 'N'.  (ta): array (m, k) = column-major
    # k x m, lda = k, 'T'.
    W.lib.check(lib.wf2hip_dgemm(b"T" if ta else b"N", b"T" if tb else b"N", m, n, k, 0.5, dp(dA), k if ta else m,
                                 dp(dB), n if tb else k, -2.0, dp(dC), ldc))
    got = dC.numpy().reshape(n, ldc).T
    C2 = Cm.reshape(n, ldc).T
    _check(got[:m, :], 0.5 * opA, opB, extra=-2.0 * C2[:m, :], what="column-major call")
    np.testing.assert_array_equal(got[m:, :], C2[m:, :])


@pytest.mark.parametrize("batch,m,n,k", [(20000, 4, 4, 4), (4096, 8, 8, 8), (300, 2, 3, 1000), (64, 16, 16, 200)])
@pytest.mark.parametrize("ta", [False, True])
@pytest.mark.parametrize("tb", [False, True])
def test_double_matmul_many_small_matrices(gpu, batch, m, n, k, ta, tb):
    """Batches of products with a few output elements each (an output element per thread, or per wavefront over
    a longer K), against the product in extended precision."""
    F = gpu.functional
    rng = np.random.default_rng(batch + m + n + k)
    A = rng.standard_normal((batch, k, m) if ta else (batch, m, k))
    B = rng.standard_normal((batch, n, k) if tb else (batch, k, n))
    a, b = D(A), D(B)
    got = F.matmul(F.t(a) if ta else a, F.t(b) if tb else b).numpy()
    opA = A.transpose(0, 2, 1) if ta else A
    opB = B.transpose(0, 2, 1) if tb else B
    want = opA @ opB
    scale = np.abs(opA) @ np.abs(opB)
    assert got.shape == (batch, m, n)
    assert np.max(np.abs(got - want) / scale) <= 8 * k * EPS
    for i in (0, batch // 2, batch - 1):
        _check(got[i], opA[i], opB[i], what=f"matrix {i}, extended precision")
