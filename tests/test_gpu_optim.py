"""Optimiser steps and the backward products on the device.

The reference's SGD and Adam are compositions of the element-wise nodes
(source/optimizers/impls/sgd.lisp:18-34, adam.lisp:45-117); every operation is
one IEEE binary32 operation, for which numpy float32 arithmetic is the closed
form (bit-identical to the reference's SIMD kernels, see
test_oracle_golden.py::test_binary_closed_form).  Bar: the node composition,
the fused kernel and numpy agree bit for bit, state included.
"""
import ctypes as C
import math

import numpy as np
import pytest

from helpers import assert_bit_equal

pytestmark = pytest.mark.gpu
f32 = np.float32


def expt(base, power):
    """(expt single-float fixnum) by squaring in single-float products.  Common Lisp leaves the
    algorithm to the implementation, so the last bit of lr_t is unpinned by the reference; the
    device step takes lr_t as a host scalar either way, and that is what is compared here."""
    total = base if power & 1 else f32(1)
    power >>= 1
    while power:
        base = f32(base * base)
        if power & 1:
            total = f32(base * total)
        power >>= 1
    return total


def numpy_adam(p, g, m, v, n, lr=1e-3, eps=1e-7, b1=0.9, b2=0.999):
    lr, eps, b1, b2 = f32(lr), f32(eps), f32(b1), f32(b2)
    lr_t = lr * (np.sqrt(f32(1) - expt(b2, n), dtype=f32) / (f32(1) - expt(b1, n)))
    m = m + (g - m) * (f32(1) - b1)
    v = v + (f32(1) - b2) * (g * g - v)
    p = p - (m * lr_t) / (eps + np.sqrt(v))
    return p, m, v


@pytest.mark.parametrize("n", [1, 3, 4, 1000, 4099, 1 << 20])
def test_sgd_step(gpu, n):
    W = gpu
    F = W.functional
    rng = np.random.default_rng(n)
    p0 = rng.standard_normal(n).astype(f32)
    g0 = rng.standard_normal(n).astype(f32)
    out = {}
    for mode in ("nodes", "fused"):
        p, g = F.from_numpy(p0), F.from_numpy(g0)
        opt = W.optimizers.SGD(p, lr=0.05, mode=mode)
        opt.step(g)
        out[mode] = (p.numpy(), g.numpy())
    gs = g0 * f32(0.05)
    assert_bit_equal(out["fused"][0], p0 - gs, "param vs numpy")
    assert_bit_equal(out["fused"][1], gs, "the gradient is scaled in place, as the reference does")
    assert_bit_equal(out["fused"][0], out["nodes"][0], "param fused vs nodes")
    assert_bit_equal(out["fused"][1], out["nodes"][1], "grad fused vs nodes")


@pytest.mark.parametrize("shape", [(7,), (33, 5), (4, 1000), (1 << 20,)])
def test_adam_steps(gpu, shape):
    W = gpu
    F = W.functional
    rng = np.random.default_rng(sum(shape))
    p0 = rng.standard_normal(shape).astype(f32)
    opts = {mode: W.optimizers.Adam(F.from_numpy(p0), mode=mode) for mode in ("nodes", "fused")}
    p, m, v = p0.copy(), np.zeros(shape, f32), np.zeros(shape, f32)
    for step in range(1, 6):
        g = (rng.standard_normal(shape) * 10.0 ** rng.integers(-3, 2)).astype(f32)
        p, m, v = numpy_adam(p, g, m, v, step)
        for mode, opt in opts.items():
            opt.step(F.from_numpy(g))
            assert_bit_equal(opt.param.numpy(), p, f"{mode} param step {step}")
            assert_bit_equal(opt.m.numpy(), m, f"{mode} m step {step}")
            assert_bit_equal(opt.v.numpy(), v, f"{mode} v step {step}")


def test_optimizer_argument_checks(gpu):
    W = gpu
    lib = W.lib.get()
    buf = W.HIPTensor([64])
    p = C.c_void_p(buf.ptr)
    q = C.c_void_p(buf.ptr + 4 * 8)
    assert lib.wf2hip_sgd_step_f32(32, p, q, 0.1) == W.lib.EOVERLAP
    assert lib.wf2hip_adam_step_f32(16, p, q, p, q, 0.1, 0.001, 1e-3, 1e-7) == W.lib.EOVERLAP
    assert lib.wf2hip_sgd_step_f32(0, p, q, 0.1) == 0
    with pytest.raises(ValueError):
        W.optimizers.SGD(buf.view((0, 32)), mode="fused").step(W.HIPTensor([32]))


def test_matmul_backward_products(gpu):
    """MatMulNode's backward (base-impl/matrix-ops.lisp:10-15): dA = dOut B^T,
    dB = A^T dOut through lazy transposes, batched, against float64."""
    F = gpu.functional
    rng = np.random.default_rng(21)
    for batch, m, k, n in [((), 37, 53, 29), ((3,), 64, 128, 96), ((2, 2), 130, 70, 33), ((), 512, 256, 384)]:
        A = rng.standard_normal(batch + (m, k)).astype(f32)
        B = rng.standard_normal(batch + (k, n)).astype(f32)
        dO = rng.standard_normal(batch + (m, n)).astype(f32)
        dA_, dB_, dO_ = F.from_numpy(A), F.from_numpy(B), F.from_numpy(dO)
        da = F.matmul(dO_, F.t(dB_)).numpy()
        db = F.matmul(F.t(dA_), dO_).numpy()
        A64, B64, dO64 = A.astype(np.float64), B.astype(np.float64), dO.astype(np.float64)
        for got, l, r in ((da, dO64, np.swapaxes(B64, -1, -2)), (db, np.swapaxes(A64, -1, -2), dO64)):
            want = l @ r
            bound = 1e-5 * (np.abs(l) @ np.abs(r))
            assert np.all(np.abs(got - want) <= bound)


def test_training_loop_converges(gpu):
    """Least squares y = x W* fitted with the device-only loop forward, backward
    products, Adam: the loss falls by four orders of magnitude."""
    W = gpu
    F = W.functional
    rng = np.random.default_rng(2)
    x = rng.standard_normal((256, 64)).astype(f32)
    w_true = rng.standard_normal((64, 32)).astype(f32)
    y = x @ w_true
    dx, dy = F.from_numpy(x), F.from_numpy(y)
    w = F.from_numpy(np.zeros((64, 32), f32))
    opt = W.optimizers.Adam(w, lr=0.05)
    losses = []
    for it in range(300):
        err = F.sub_(F.matmul(dx, w), dy)                 # (256, 32)
        grad = F.mul_(F.matmul(F.t(dx), err), 2.0 / 256)  # d/dW mean squared error
        opt.step(grad)
        if it % 50 == 0 or it == 299:
            losses.append(float(np.mean(err.numpy() ** 2)))
    assert losses[-1] < 1e-4 * losses[0], losses


def test_weights_round_trip(gpu, tmp_path):
    """.npy and :wf2model I/O (examples/gpt-2/utils.lisp:6-9,
    backends/lisp/wf2model.lisp:5-54): bit-exact round trips, views saved as
    seen, storage vectors saved flat, non-float files refused."""
    import json
    W = gpu
    rng = np.random.default_rng(1)
    a = rng.standard_normal((5, 7, 3)).astype(f32)
    np.save(tmp_path / "a.npy", a)
    t = W.io.load_npy(str(tmp_path / "a.npy"))
    assert t.shape == [5, 7, 3]
    assert_bit_equal(t.numpy(), a, "load_npy")
    W.io.save_npy(t.view((1, 4), True, 2), str(tmp_path / "v.npy"))
    assert_bit_equal(np.load(tmp_path / "v.npy"), a[1:4, :, 2:3], "save_npy of a view")
    np.save(tmp_path / "i.npy", np.arange(4))
    with pytest.raises(TypeError):
        W.io.load_npy(str(tmp_path / "i.npy"))
    np.save(tmp_path / "d.npy", a.astype(np.float64))
    assert_bit_equal(W.io.load_npy(str(tmp_path / "d.npy")).numpy(), a, "float64 file narrows to float")
    state = {"layer/w": t, "bias": W.HIPTensor.from_numpy(a[0, 0]), "steps": 12, "lr": 0.5}
    W.io.save_weights(str(tmp_path / "model"), state)
    table = json.load(open(tmp_path / "model" / "parameters.json"))
    assert table["steps"] == 12 and table["layer/w"].endswith("layer/w.npy")
    assert np.load(table["layer/w"]).shape == (105,)      # the storage vector, flat
    back = W.io.load_weights(str(tmp_path / "model"), shapes={"layer/w": (5, 7, 3)})
    assert back["steps"] == 12 and back["lr"] == 0.5
    assert_bit_equal(back["layer/w"].numpy(), a, "wf2model tensor")
    assert_bit_equal(back["bias"].numpy(), a[0, 0], "wf2model flat tensor")


@pytest.mark.parametrize("fused_loss", [False, True])
def test_classifier_training_step_by_step(gpu, fused_loss):
    """A two-layer classifier trained entirely on the device with the
    reference's recipes: Linear = matmul + bias (AddNode with a broadcast row),
    !relu = x * (x > 0), Softmax-Cross-Entropy-Node forward and backward
    (nn/criterion.lisp:82-126), bias gradients as !sum over the batch, matmul
    backward products, Adam.  Every step is compared with the same recipe in
    float64 on the host (loss and weights), and the loss must fall.  With
    `fused_loss` the criterion is HIP-Softmax-Cross-Entropy-Node and its one-kernel
    backward instead of the node compositions."""
    W = gpu
    F = W.functional
    nn = W.nn
    rng = np.random.default_rng(33)
    n, d, h, c = 512, 96, 128, 10
    centers = rng.standard_normal((c, d)) * 2.0
    cls = rng.integers(0, c, n)
    x = (centers[cls] + rng.standard_normal((n, d))).astype(f32)
    labels = np.eye(c, dtype=f32)[cls]
    params = {"w1": (rng.standard_normal((d, h)) * 0.1).astype(f32), "b1": np.zeros((1, h), f32),
              "w2": (rng.standard_normal((h, c)) * 0.1).astype(f32), "b2": np.zeros((1, c), f32)}
    dev = {k: F.from_numpy(v) for k, v in params.items()}
    opt = {k: W.optimizers.Adam(dev[k], lr=0.01) for k in dev}
    dx, dl = F.from_numpy(x), F.from_numpy(labels)

    # float64 mirror of the same recipe (mean-subtracted softmax as the reference's !softmax)
    ref = {k: v.astype(np.float64) for k, v in params.items()}
    state = {k: (np.zeros_like(v), np.zeros_like(v)) for k, v in ref.items()}

    def host_step(t):
        a1 = x @ ref["w1"] + ref["b1"]
        h1 = a1 * (a1 > 0)
        a2 = h1 @ ref["w2"] + ref["b2"]
        e = np.exp(a2 - a2.mean(axis=1, keepdims=True))
        z = e / e.sum(axis=1, keepdims=True)
        loss = np.mean(-labels * np.log(z + 1e-7))
        dz = (z - labels) * (1.0 / labels.size) / n  # d mean / d out, then sce-diff-static: / batch
        grads = {"w2": h1.T @ dz, "b2": dz.sum(axis=0, keepdims=True)}
        dh = (dz @ ref["w2"].T) * (a1 > 0)
        grads["w1"], grads["b1"] = x.T @ dh, dh.sum(axis=0, keepdims=True)
        for k, g in grads.items():
            m, v = state[k]
            m += (g - m) * (1 - 0.9)
            v += (1 - 0.999) * (g * g - v)
            lr_t = 0.01 * np.sqrt(1 - 0.999 ** t) / (1 - 0.9 ** t)
            ref[k] -= (m * lr_t) / (1e-7 + np.sqrt(v))
        return loss

    losses = []
    for t in range(1, 41):
        a1 = F.add(F.matmul(dx, dev["w1"]), dev["b1"])
        mask = F.where(a1, ">", 0.0)
        h1 = F.mul(a1, mask)
        a2 = F.add(F.matmul(h1, dev["w2"]), dev["b2"])
        if fused_loss:
            loss, z = nn.softmax_cross_entropy_fused(a2, dl, reduction="mean")
            dz = nn.softmax_cross_entropy_backward_fused(1.0 / labels.size, z, dl)
        else:
            loss, z = nn.softmax_cross_entropy(a2, dl, avoid_overflow=True, reduction="mean")
            dz = nn.softmax_cross_entropy_backward(1.0 / labels.size, z, dl)
        grads = {"w2": F.matmul(F.t(h1), dz), "b2": F.sum(dz, axis=0)}  # (1, c): the reduced axis stays, size 1
        dh = F.mul_(F.matmul(dz, F.t(dev["w2"])), mask)
        grads["w1"], grads["b1"] = F.matmul(F.t(dx), dh), F.sum(dh, axis=0)
        for k in dev:
            opt[k].step(grads[k])
        want = host_step(t)
        got = float(loss.numpy().ravel()[0])
        losses.append(got)
        assert abs(got - want) <= 2e-4 * abs(want) + 1e-6, (t, got, want)
    for k in dev:
        np.testing.assert_allclose(dev[k].numpy(), ref[k], rtol=0, atol=5e-3, err_msg=k)
    assert losses[-1] < 0.5 * losses[0], losses
