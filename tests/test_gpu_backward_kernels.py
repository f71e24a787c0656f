"""The one-kernel backward forms (activation gradients, softmax and causal softmax gradients,
LayerNorm gradients) against float64 closed forms and against their node compositions."""
import importlib

import numpy as np
import pytest

from helpers import assert_bit_equal

pytestmark = pytest.mark.gpu
f32 = np.float32


def test_activation_backward_bits_of_the_compositions(gpu):
    """ReLU, leaky ReLU and sigmoid gradients are the binary32 operations of the composed recipes
    (A>scal / A>=scal masks, s (1 - s) with s from the sigmoid kernel) times dout: bit-identical."""
    W = gpu
    F = W.functional
    rng = np.random.default_rng(41)
    x = (rng.standard_normal((37, 1001)) * 3).astype(f32)
    x.flat[:6] = [0.0, -0.0, np.inf, -np.inf, 1e-40, -1e-40]
    d = rng.standard_normal(x.shape).astype(f32)
    dx, dd = F.from_numpy(x), F.from_numpy(d)
    assert_bit_equal(F.activation_backward("relu", dx, dd).numpy(), d * (x > 0).astype(f32), "relu")
    assert_bit_equal(F.activation_backward("leaky_relu", dx, dd, p=0.01).numpy(),
                     d * np.where(x >= 0, f32(1), f32(0.01)), "leaky relu")
    s = F.sigmoid_fused(dx)
    want = F.mul(dd, F.mul(s, F.sub(1.0, s))).numpy()
    assert_bit_equal(F.activation_backward("sigmoid", dx, dd).numpy(), want, "sigmoid")
    assert_bit_equal(dd.numpy(), d, "dout untouched when not in place")
    # in place, on a strided window of a larger tensor, x a transposed view
    big = rng.standard_normal((64, 200)).astype(f32)
    xt = (rng.standard_normal((100, 64)) * 2).astype(f32)
    t = F.from_numpy(big)
    win = t.view(True, (50, 150))
    F.activation_backward("relu", F.from_numpy(xt).permute(1, 0), win, in_place=True)
    want = big.copy()
    want[:, 50:150] *= (xt.T > 0)
    assert_bit_equal(t.numpy(), want, "relu in place on a window, transposed x")


def test_gelu_backward_against_float64(gpu):
    from test_math_cpu import gelu_grad_truth
    W = gpu
    F = W.functional
    rng = np.random.default_rng(42)
    x = np.concatenate([rng.uniform(-10, 10, 1 << 20), rng.standard_normal(1 << 20) * 2,
                        [0.0, -0.0, 40.0, -40.0]]).astype(f32)
    d = rng.standard_normal(x.size).astype(f32)
    got = F.activation_backward("gelu", F.from_numpy(x), F.from_numpy(d)).numpy().astype(np.float64)
    ends = F.activation_backward("gelu", F.from_numpy(np.array([np.inf, -np.inf, np.nan], f32)),
                                 F.from_numpy(np.array([3.0, 3.0, 3.0], f32))).numpy()
    assert ends[0] == 3.0 and ends[1] == 0.0 and np.isnan(ends[2])
    g, mag = gelu_grad_truth(x)
    # v_exp_f32 returns 0 below 2^-126: gradients under about 2^-120 are flushed, an absolute floor
    ratio = np.abs(got - d * g) / (np.abs(d) * (mag + 2.0 ** -120 / 1e-6))
    assert ratio[np.abs(x) <= 4].max() <= 1.2e-6 and ratio.max() <= 1e-5
    # against the node composition of the derivative (an absolute comparison: the composition
    # cancels in 1 + tanh on the left)
    xs = (rng.standard_normal((64, 300)) * 2).astype(f32)
    ds = rng.standard_normal(xs.shape).astype(f32)
    comp = F.mul(F.from_numpy(ds), F.gelu_derivative(F.from_numpy(xs))).numpy()
    one = F.activation_backward("gelu", F.from_numpy(xs), F.from_numpy(ds)).numpy()
    assert np.max(np.abs(comp - one)) <= 1e-6 * np.max(np.abs(ds))


def _softmax_bwd_truth(y, dy, scale, causal):
    y, dy = y.astype(np.float64), dy.astype(np.float64)
    if causal:
        keep = np.tril(np.ones(y.shape[-2:], bool))
        dy = np.where(keep, dy, 0.0)
    dot = (dy * y).sum(-1, keepdims=True)
    return scale * y * (dy - dot), np.abs(scale) * np.abs(y) * (np.abs(dy) + np.abs(dy * y).sum(-1, keepdims=True))


@pytest.mark.parametrize("rows,cols", [(16384, 1), (16385, 2), (20001, 10), (16500, 31), (16384, 32), (16400, 33), (16390, 64), (5, 7), (33, 256), (100, 1000), (64, 1024), (17, 1537), (9, 2048), (6, 5000),
                                       (7, 2049), (5, 4096), (9, 8193), (4, 16385), (3, 32768), (3, 50257), (1, 1 << 21), (300, 8192),
                                       (300, 40001), (2, 1234567)])
def test_softmax_backward_rows(gpu, rows, cols):
    W = gpu
    F = W.functional
    rng = np.random.default_rng(rows * 10007 + cols)
    logits = (rng.standard_normal((rows, cols)) * 3).astype(f32)
    y = F.softmax_fused(F.from_numpy(logits))
    dy = rng.standard_normal((rows, cols)).astype(f32)
    want, mag = _softmax_bwd_truth(y.numpy(), dy, 1.0, False)
    got = F.softmax_backward(y, F.from_numpy(dy))
    assert np.max(np.abs(got.numpy() - want) / (mag + 1e-30)) <= 2e-6
    comp = F.softmax_backward_composed(y, F.from_numpy(dy))
    assert np.max(np.abs(got.numpy() - comp.numpy()) / (mag + 1e-30)) <= 2e-6
    # in place, with a scale
    d2 = F.from_numpy(dy)
    out = F.softmax_backward(y, d2, scale=0.37, in_place=True)
    assert out is d2
    assert np.max(np.abs(d2.numpy() - 0.37 * want) / (mag + 1e-30)) <= 2e-6


@pytest.mark.parametrize("batch,seq", [(3, 5), (4, 70), (2, 256), (2, 1000), (1, 1024)])
def test_causal_softmax_backward(gpu, batch, seq):
    """Above the diagonal dout is never read (NaN there must not spread) and dx is exactly 0."""
    W = gpu
    F = W.functional
    rng = np.random.default_rng(seq)
    s = (rng.standard_normal((batch, seq, seq)) * 2).astype(f32)
    y = F.causal_softmax_fused(F.from_numpy(s), 0.125)
    dy = rng.standard_normal((batch, seq, seq)).astype(f32)
    dy[:, np.triu_indices(seq, 1)[0], np.triu_indices(seq, 1)[1]] = np.nan
    want, mag = _softmax_bwd_truth(y.numpy(), np.nan_to_num(dy), 0.125, True)
    got = F.softmax_backward(y, F.from_numpy(dy), scale=0.125, causal=True).numpy()
    assert np.all(np.isfinite(got))
    upper = np.triu(np.ones((seq, seq), bool), 1)
    assert np.all(got[:, upper] == 0.0)
    assert np.max(np.abs(got - want) / (mag + 1e-30)) <= 2e-6
    with pytest.raises(Exception):
        F.softmax_backward(F.from_numpy(np.zeros((2, 3, 4), f32)), F.from_numpy(np.zeros((2, 3, 4), f32)), causal=True)


@pytest.mark.parametrize("rows,cols", [(1, 4), (5, 60), (37, 768), (1000, 1024), (300, 2048), (4099, 768),
                                       (257, 1001), (8192, 768),
                                       # beyond 2048 columns: a workgroup per row, 3 ... 8 vectors per thread
                                       (6, 2052), (700, 3072), (33, 4096), (1100, 5120), (5, 6148), (600, 8192),
                                       # 8196 ... 16384 columns and at least a row per compute unit: the same with 1024 threads
                                       (300, 16384), (260, 9000), (513, 12292),
                                       # very many rows of at most 64 columns: a thread per row
                                       (16384, 10), (20001, 33), (16400, 64), (16385, 5), (40000, 32)])
def test_layernorm_backward(gpu, rows, cols):
    from oracle import gpt2_block_ref as ref
    W = gpu
    F = W.functional
    rng = np.random.default_rng(rows + 31 * cols)
    x = (rng.standard_normal((rows, cols)) * 2 + 0.5).astype(f32)
    g = (1 + 0.2 * rng.standard_normal(cols)).astype(f32)
    dy = rng.standard_normal((rows, cols)).astype(f32)
    eps = 1e-5
    dx, dg, db, mag, mag_g = ref.layer_norm_backward(x.astype(np.float64), g.astype(np.float64), dy.astype(np.float64), eps)
    gx, gg, gb = F.layer_norm_backward(F.from_numpy(x), F.from_numpy(g), F.from_numpy(dy), eps)
    assert gx.shape == [rows, cols] and gg.shape == [cols] and gb.shape == [cols]
    assert np.max(np.abs(gx.numpy() - dx) / mag) <= 3e-6
    assert np.max(np.abs(gg.numpy() - dg) / (mag_g + 1e-30)) <= 3e-6
    assert np.max(np.abs(gb.numpy() - db) / (np.abs(dy).sum(0) + 1e-30)) <= 1e-6
    if rows <= 1000:
        cx, cg, cb = F.layer_norm_backward_composed(F.from_numpy(x), F.from_numpy(g), F.from_numpy(dy), eps)
        assert np.max(np.abs(cx.numpy() - gx.numpy()) / mag) <= 5e-6
        assert np.max(np.abs(cg.numpy() - gg.numpy()) / (mag_g + 1e-30)) <= 5e-6


@pytest.mark.parametrize("rows,cols,shift", [(6, 8196, 0), (6, 4098, 0), (3, 16384, 0), (2, 40001, 0), (1, 262144 + 8, 0),
                                             (700, 8200, 0), (1100, 2050, 0), (5, 32768, 1), (4, 3072, 3)])
def test_layernorm_backward_in_pieces(gpu, rows, cols, shift):
    """More than 8192 columns, or more than 2048 that cannot be read with 16-byte loads (a column count that is no
    multiple of 4, or tensors `shift` elements off a 16-byte boundary): the row in pieces of 16384 columns over several
    workgroups, through the C ABI, against binary64 and against the node composition."""
    from oracle import gpt2_block_ref as ref
    import ctypes as C
    W = gpu
    F = W.functional
    rng = np.random.default_rng(rows + 7 * cols)
    x = (rng.standard_normal((rows, cols)) * 2 + 0.5).astype(f32)
    g = (1 + 0.1 * rng.standard_normal(cols)).astype(f32)
    dy = rng.standard_normal((rows, cols)).astype(f32)
    lib = W.lib.get()
    total = rows * cols
    hold = [F.from_numpy(np.concatenate([np.zeros(shift, f32), a.ravel()])) for a in (x, g, dy)]
    outs = [W.HIPTensor([n + shift]) for n in (total, cols, cols)]
    p = lambda t: C.c_void_p(t.ptr + 4 * shift)  # noqa: E731
    rc = lib.wf2hip_layernorm_backward_f32(rows, cols, p(hold[0]), p(hold[1]), p(hold[2]), 1e-5, p(outs[0]), p(outs[1]),
                                           p(outs[2]))
    assert rc == 0
    gx = outs[0].numpy()[shift:].reshape(rows, cols)
    gg, gb = outs[1].numpy()[shift:], outs[2].numpy()[shift:]
    dx, dg, db, mag, mag_g = ref.layer_norm_backward(x.astype(np.float64), g.astype(np.float64), dy.astype(np.float64), 1e-5)
    assert np.max(np.abs(gx - dx) / mag) <= 3e-6
    # xhat comes from x - (float)mean: where x is close to the mean the rounding of the mean (6e-8 |mean| rstd, about
    # 1.5e-8 here) is large against |xhat| itself, and with a row or two nothing averages it out
    assert np.max(np.abs(gg - dg) / (mag_g + 0.03 * np.abs(dy).sum(0) + 1e-30)) <= 3e-6
    assert np.max(np.abs(gb - db) / (np.abs(dy).sum(0) + 1e-30)) <= 1e-6
    if total <= 1 << 20:
        cx, cg, cb = F.layer_norm_backward_composed(F.from_numpy(x), F.from_numpy(g), F.from_numpy(dy), 1e-5)
        assert np.max(np.abs(cx.numpy() - gx) / mag) <= 5e-6
        assert np.max(np.abs(cg.numpy() - gg) / (mag_g + 0.03 * np.abs(dy).sum(0) + 1e-30)) <= 5e-6
    # dx may be dy
    rc = lib.wf2hip_layernorm_backward_f32(rows, cols, p(hold[0]), p(hold[1]), p(hold[2]), 1e-5, p(hold[2]), p(outs[1]),
                                           p(outs[2]))
    assert rc == 0
    assert np.array_equal(hold[2].numpy()[shift:].reshape(rows, cols), gx)
    assert np.array_equal(outs[1].numpy()[shift:], gg)


def test_backward_entries_on_empty_operands(gpu):
    """Zero rows, zero columns, zero elements: nothing is launched, column sums of no rows are 0."""
    import ctypes as C
    W = gpu
    lib = W.lib.get()
    p = lambda t: C.c_void_p(t.ptr)  # noqa: E731
    a, b, c = (W.HIPTensor([4, 8], initial_element=3.0) for _ in range(3))
    g = W.HIPTensor([8], initial_element=1.0)
    dg, db = W.HIPTensor([8], initial_element=5.0), W.HIPTensor([8], initial_element=5.0)
    assert lib.wf2hip_softmax_backward_rows_f32(0, 8, p(a), 8, p(b), 8, p(c), 8, 1.0, 0) == 0
    assert lib.wf2hip_softmax_backward_rows_f32(4, 0, p(a), 8, p(b), 8, p(c), 8, 1.0, 0) == 0
    assert lib.wf2hip_layernorm_backward_f32(0, 8, p(a), p(g), p(b), 1e-5, p(c), p(dg), p(db)) == 0
    assert np.all(dg.numpy() == 0.0) and np.all(db.numpy() == 0.0)
    assert np.all(c.numpy() == 3.0)
    v = W.lib.View2()
    v.rank = 1
    v.shape[0] = 0
    v.stride_a[0] = v.stride_b[0] = 1
    assert lib.wf2hip_activation_backward_nd(W.lib.GELU, C.byref(v), p(a), p(b), 0.0) == 0
    assert lib.wf2hip_activation_backward_nd(7, C.byref(v), p(a), p(b), 0.0) == 0  # nothing to do, nothing checked
    v.shape[0] = 8
    assert lib.wf2hip_activation_backward_nd(7, C.byref(v), p(a), p(b), 0.0) == W.lib.EINVAL  # not an activation
    # pitches smaller than the row, a causal form that is not square
    assert lib.wf2hip_softmax_backward_rows_f32(4, 8, p(a), 4, p(b), 8, p(c), 8, 1.0, 0) == W.lib.EINVAL
    assert lib.wf2hip_softmax_backward_rows_f32(4, 8, p(a), 8, p(b), 8, p(c), 8, 1.0, 4) == W.lib.EINVAL
    # dx over y
    assert lib.wf2hip_softmax_backward_rows_f32(4, 8, p(a), 8, p(b), 8, p(a), 8, 1.0, 0) == W.lib.EOVERLAP
