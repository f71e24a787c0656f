"""The float64 backward of the transformer block (the checker of the device backward) against what
the mathematics fixes: central differences of the float64 forward along random directions, for the
input and every parameter, on a small block with non-trivial LayerNorm parameters and biases."""
import numpy as np

from oracle import gpt2_block_ref as ref


def _params(rng, d, ff):
    w = lambda *s: rng.standard_normal(s) * 0.2  # noqa: E731
    return {"w_qkv": w(d, 3 * d), "w_o": w(d, d), "w_fc": w(d, ff), "w_proj": w(ff, d),
            "b_qkv": w(3 * d), "b_o": w(d), "b_fc": w(ff), "b_proj": w(d),
            "ln1_g": 1 + w(d), "ln1_b": w(d), "ln2_g": 1 + w(d), "ln2_b": w(d)}


def test_block_backward_matches_central_differences():
    rng = np.random.default_rng(7)
    B, T, d, H, ff = 2, 9, 12, 3, 20
    p = _params(rng, d, ff)
    x = rng.standard_normal((B, T, d))
    dout = rng.standard_normal((B, T, d))
    grads, scales = ref.block_backward(x, p, H, dout, eps=1e-5)
    loss = lambda xx, pp: float((ref.block_forward(xx, pp, H, eps=1e-5) * dout).sum())  # noqa: E731
    h = 1e-5
    for name in ["x"] + sorted(p):
        for trial in range(3):
            base = x if name == "x" else p[name]
            direction = rng.standard_normal(base.shape)
            plus, minus = dict(p), dict(p)
            if name == "x":
                numeric = (loss(x + h * direction, p) - loss(x - h * direction, p)) / (2 * h)
            else:
                plus[name] = base + h * direction
                minus[name] = base - h * direction
                numeric = (loss(x, plus) - loss(x, minus)) / (2 * h)
            analytic = float((grads[name] * direction).sum())
            bound = float((scales[name] * np.abs(direction)).sum())
            assert abs(numeric - analytic) <= 1e-7 * bound + 1e-9, (name, trial, numeric, analytic)
        # the yardstick dominates the gradient it belongs to
        assert np.all(np.abs(grads[name]) <= scales[name] * (1 + 1e-12) + 1e-300), name


def test_gelu_derivative_closed_form():
    x = np.linspace(-6, 6, 2001)
    h = 1e-6
    numeric = (ref.gelu(x + h) - ref.gelu(x - h)) / (2 * h)
    assert np.max(np.abs(numeric - ref.gelu_derivative(x))) < 1e-9
    assert ref.gelu_derivative(np.array([0.0]))[0] == 0.5


def test_layer_norm_backward_rows_sum_to_zero():
    """dx of LayerNorm is orthogonal to the constant vector and to xh (shift and scale invariance)."""
    rng = np.random.default_rng(3)
    x = rng.standard_normal((5, 16))
    g = 1 + 0.1 * rng.standard_normal(16)
    dout = rng.standard_normal((5, 16))
    dx, dg, db, mag, mag_g = ref.layer_norm_backward(x, g, dout, 0.0)
    assert np.max(np.abs(dx.sum(axis=-1))) < 1e-12
    xh = (x - x.mean(-1, keepdims=True)) / x.std(-1, keepdims=True)
    assert np.max(np.abs((dx * xh).sum(axis=-1))) < 1e-12
    assert np.all(np.abs(dx) <= mag + 1e-15) and np.all(np.abs(dg) <= mag_g + 1e-15)
