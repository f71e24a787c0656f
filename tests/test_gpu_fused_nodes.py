"""The define-op nodes of the fused block through the Python mirror (the same node names
and the same library calls as lisp/fusion.lisp): HIP-Linear-Node / -Residual-Node against
the node-for-node composition and float64, HIP-Causal-Softmax-Node against the masked
softmax, the composed backward of HIP-LayerNorm-Node against the closed-form gradients,
and the argument checks of the row kernels."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def test_linear_nodes_against_composition_and_float64(gpu):
    W = gpu
    F = W.functional
    rng = np.random.default_rng(21)
    for lead, k, n in [((64,), 96, 160), ((4, 50), 768, 256), ((3, 7, 5), 40, 33)]:
        X = rng.standard_normal(lead + (k,)).astype(np.float32)
        Wt = (rng.standard_normal((k, n)) * 0.05).astype(np.float32)
        b = rng.standard_normal(n).astype(np.float32)
        R = rng.standard_normal(lead + (n,)).astype(np.float32)
        x, w, bb, r = (F.from_numpy(a) for a in (X, Wt, b, R))
        z64 = X.astype(np.float64) @ Wt.astype(np.float64) + b
        mag = np.abs(X).astype(np.float64) @ np.abs(Wt).astype(np.float64) + np.abs(b)
        plain = F.linear(x, w, bb).numpy()
        assert plain.shape == lead + (n,)
        assert np.all(np.abs(plain - z64) <= 1e-5 * mag)
        composed = F.add_(F.matmul(x, w), bb).numpy()          # MatMulNode + AddNode
        assert np.all(np.abs(plain - composed) <= 2e-5 * mag)
        res = F.linear(x, w, bb, residual=r).numpy()
        assert np.all(np.abs(res - (z64 + R)) <= 1e-5 * (mag + np.abs(R)))
        g = F.linear(x, w, bb, activation="gelu").numpy()
        want = z64 / (1.0 + np.exp(-2.0 * 0.7978845608028654 * (z64 + 0.044715 * z64 ** 3)))
        np.testing.assert_allclose(g, want, rtol=1e-4, atol=2e-5 * mag.max())
    with pytest.raises(ValueError):
        F.linear(x, w, bb, activation="gelu", residual=r)
    with pytest.raises(ValueError):
        F.linear(x, w, bb, activation="relu")


def test_causal_softmax_node(gpu):
    W = gpu
    F = W.functional
    rng = np.random.default_rng(22)
    for lead, T in [((6,), 64), ((2, 3), 100), ((1,), 1024)]:
        S = rng.standard_normal(lead + (T, T)).astype(np.float32) * 3
        got = F.causal_softmax_fused(F.from_numpy(S), scale=0.125).numpy()
        s64 = np.where(np.tril(np.ones((T, T), bool)), S.astype(np.float64) * 0.125, -np.inf)
        e = np.exp(s64 - s64.max(axis=-1, keepdims=True))
        want = e / e.sum(axis=-1, keepdims=True)
        np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-9)
        assert np.all(got[..., ~np.tril(np.ones((T, T), bool))] == 0.0)


def test_layer_norm_backward_composition(gpu):
    """The gradients HIP-LayerNorm-Node's backward composes, against the closed form in float64."""
    W = gpu
    F = W.functional
    rng = np.random.default_rng(23)
    for rows, cols in [(37, 64), (128, 768), (5, 1000)]:
        X = (rng.standard_normal((rows, cols)) * 2 + 0.3).astype(np.float32)
        g = (1 + 0.1 * rng.standard_normal(cols)).astype(np.float32)
        dY = rng.standard_normal((rows, cols)).astype(np.float32)
        dx, dg, db = F.layer_norm_backward(F.from_numpy(X), F.from_numpy(g), F.from_numpy(dY), eps=1e-5)
        x64, g64, d64 = X.astype(np.float64), g.astype(np.float64), dY.astype(np.float64)
        mu = x64.mean(axis=1, keepdims=True)
        rstd = 1.0 / np.sqrt(((x64 - mu) ** 2).mean(axis=1, keepdims=True) + 1e-5)
        xh = (x64 - mu) * rstd
        dyh = d64 * g64
        want_dx = rstd * (dyh - dyh.mean(axis=1, keepdims=True) - xh * (dyh * xh).mean(axis=1, keepdims=True))
        np.testing.assert_allclose(dx.numpy(), want_dx, rtol=2e-4, atol=2e-5)
        np.testing.assert_allclose(dg.numpy(), (d64 * xh).sum(axis=0), rtol=2e-4, atol=2e-4)
        np.testing.assert_allclose(db.numpy(), d64.sum(axis=0), rtol=1e-5, atol=1e-4)
        # and the closed form really is the derivative: a directional finite difference in float64
        def f(xv):
            m = xv.mean(axis=1, keepdims=True)
            return ((xv - m) / np.sqrt(((xv - m) ** 2).mean(axis=1, keepdims=True) + 1e-5) * g64 * d64).sum()
        v = rng.standard_normal((rows, cols))
        h = 1e-6
        assert abs((f(x64 + h * v) - f(x64 - h * v)) / (2 * h) - (want_dx * v).sum()) <= 1e-5 * abs((want_dx * v).sum()) + 1e-6


def test_row_kernels_refuse_views(gpu):
    """softmax_fused / layer_norm_fused hand base pointers to the row kernels: an `out` (or
    gamma / beta) that is a view, has another shape or another dtype must be refused, not
    written or read at the wrong address."""
    W = gpu
    F = W.functional
    x = F.from_numpy(np.random.default_rng(1).standard_normal((8, 32)).astype(np.float32))
    g = F.from_numpy(np.ones(32, np.float32))
    big = W.HIPTensor([8, 64])
    with pytest.raises(ValueError):
        F.softmax_fused(x, out=big.view(True, (0, 32)))
    with pytest.raises(ValueError):
        F.softmax_fused(x, out=W.HIPTensor([4, 64]))
    with pytest.raises(ValueError):
        F.layer_norm_fused(x, g, g, out=big.view(True, (32, 64)))
    wide = F.from_numpy(np.ones(64, np.float32))
    with pytest.raises(ValueError):
        F.layer_norm_fused(x, wide.view((16, 48)), g)
    with pytest.raises(ValueError):
        F.layer_norm_fused(x, g, F.from_numpy(np.ones(32), dtype="double"))
    assert np.all(big.numpy() == 0.0)
    ok = F.softmax_fused(x, out=W.HIPTensor([8, 32], initial_element=None)).numpy()
    assert np.allclose(ok.sum(axis=1), 1.0, atol=1e-6)
