"""The CNN of the reference's MNIST example trained on the device, step by step against float64.

examples/mnist/cnn.lisp:6-16: Conv2D(1 -> 4, 3x3), !relu, MaxPool2D(2x2), Conv2D(4 -> 16, 5x5), !relu,
MaxPool2D(2x2), reshape to (N, 16*4*4), LinearLayer(256 -> 10); criterion softmax-cross-entropy, optimiser
Adam.  Forward and backward are the compositions the reference's nodes derive (nn.py), on synthetic digits
(no dataset here).  The float64 mirror below is written independently of them, from the definitions of
convolution and pooling (windows by numpy's sliding_window_view), and is itself pinned by central
differences of its loss."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu
f32 = np.float32
sw = np.lib.stride_tricks.sliding_window_view


# ---- float64 mirror ---------------------------------------------------------------------------------
def conv_fwd(x, w, b):
    win = sw(x, w.shape[2:], axis=(2, 3))                       # N C h w kh kw
    return np.einsum("nchwij,ocij->nohw", win, w) + b[None, :, None, None]


def conv_bwd(x, w, dy):
    win = sw(x, w.shape[2:], axis=(2, 3))
    dw = np.einsum("nchwij,nohw->ocij", win, dy)
    dx = np.zeros_like(x)
    kh, kw = w.shape[2:]
    h, wd = dy.shape[2:]
    for i in range(kh):
        for j in range(kw):
            dx[:, :, i:i + h, j:j + wd] += np.einsum("nohw,oc->nchw", dy, w[:, :, i, j])
    return dx, dw, dy.sum(axis=(0, 2, 3))


def pool_fwd(x):                                                # 2x2, stride 2, floor
    h, w = x.shape[2] // 2, x.shape[3] // 2
    win = x[:, :, :2 * h, :2 * w].reshape(x.shape[0], x.shape[1], h, 2, w, 2)
    return win.max(axis=(3, 5))


def pool_bwd(x, dy):
    h, w = x.shape[2] // 2, x.shape[3] // 2
    win = x[:, :, :2 * h, :2 * w].reshape(x.shape[0], x.shape[1], h, 2, w, 2)
    mask = win == win.max(axis=(3, 5), keepdims=True)           # every maximum of a window receives dout
    dx = np.zeros_like(x)
    dx[:, :, :2 * h, :2 * w] = (mask * dy[:, :, :, None, :, None]).reshape(x.shape[0], x.shape[1], 2 * h, 2 * w)
    return dx


def model_loss_and_grads(p, x, labels, want_grads=True, node_divides_by_batch=True):
    """The loss and its gradients.  Softmax-Cross-Entropy-Node's backward divides by the batch size on top of
    what the mean has already divided by (sce-diff-static, source/nn/criterion.lisp:82-88, 103-110), so the
    gradients the reference trains with are the derivatives of the loss over N; `node_divides_by_batch=False`
    gives the derivatives themselves (what central differences measure)."""
    a1 = conv_fwd(x, p["w1"], p["b1"])
    r1 = a1 * (a1 > 0)
    p1 = pool_fwd(r1)
    a2 = conv_fwd(p1, p["w2"], p["b2"])
    r2 = a2 * (a2 > 0)
    p2 = pool_fwd(r2)
    flat = p2.reshape(x.shape[0], -1)
    logits = flat @ p["w3"].T + p["b3"]
    e = np.exp(logits - logits.max(axis=1, keepdims=True))
    z = e / e.sum(axis=1, keepdims=True)
    loss = np.mean(-labels * np.log(z + np.float64(f32(1e-7))))
    if not want_grads:
        return loss
    n = x.shape[0]
    dlogits = (z - labels) * (1.0 / labels.size) / (n if node_divides_by_batch else 1.0)
    g = {"w3": dlogits.T @ flat, "b3": dlogits.sum(axis=0)}
    dp2 = (dlogits @ p["w3"]).reshape(p2.shape)
    da2 = pool_bwd(r2, dp2) * (a2 > 0)
    dp1, g["w2"], g["b2"] = conv_bwd(p1, p["w2"], da2)
    da1 = pool_bwd(r1, dp1) * (a1 > 0)
    _, g["w1"], g["b1"] = conv_bwd(x, p["w1"], da1)
    return loss, g


def _digits(rng, n):
    """Ten fixed 28 x 28 prototypes plus noise: enough structure for the loss to fall."""
    protos = rng.standard_normal((10, 1, 28, 28))
    protos = sw(np.pad(protos, ((0, 0), (0, 0), (2, 2), (2, 2))), (5, 5), axis=(2, 3)).mean(axis=(4, 5))  # smoothed
    cls = rng.integers(0, 10, n)
    x = protos[cls] * 3.0 + 0.5 * rng.standard_normal((n, 1, 28, 28))
    return x.astype(f32), np.eye(10, dtype=f32)[cls]


def _params(rng):
    return {"w1": (rng.standard_normal((4, 1, 3, 3)) * 0.3).astype(f32), "b1": np.zeros(4, f32),
            "w2": (rng.standard_normal((16, 4, 5, 5)) * 0.1).astype(f32), "b2": np.zeros(16, f32),
            "w3": (rng.standard_normal((10, 256)) * 0.05).astype(f32), "b3": np.zeros(10, f32)}


def test_float64_mirror_by_central_differences():
    rng = np.random.default_rng(3)
    x, labels = _digits(rng, 6)
    p = {k: v.astype(np.float64) for k, v in _params(rng).items()}
    x = x.astype(np.float64)
    _, g = model_loss_and_grads(p, x, labels, node_divides_by_batch=False)
    for name in p:
        for _ in range(3):
            at = tuple(rng.integers(0, s) for s in p[name].shape)
            h = 1e-6
            hi, lo = {k: v.copy() for k, v in p.items()}, {k: v.copy() for k, v in p.items()}
            hi[name][at] += h
            lo[name][at] -= h
            num = (model_loss_and_grads(hi, x, labels, False) - model_loss_and_grads(lo, x, labels, False)) / (2 * h)
            assert abs(num - g[name][at]) <= 1e-8 + 1e-5 * abs(num), (name, at, num, g[name][at])


def _device_step(W, dev, dx, dl, n, fused_loss):
    F, nn = W.functional, W.nn
    a1 = nn.conv2d(dx, dev["w1"], dev["b1"])
    m1 = F.where(a1, ">", 0.0)
    r1 = F.mul(a1, m1)
    p1 = nn.max_pool2d(r1, 2)
    a2 = nn.conv2d(p1, dev["w2"], dev["b2"])
    m2 = F.where(a2, ">", 0.0)
    r2 = F.mul(a2, m2)
    p2 = nn.max_pool2d(r2, 2)
    flat = F.reshape(p2, n, -1)
    logits = F.add(F.matmul(flat, F.t(dev["w3"])), F.reshape(dev["b3"], 1, -1))   # LinearLayer: x . W^T + b
    if fused_loss:
        loss, z = nn.softmax_cross_entropy_fused(logits, dl, reduction="mean")
        dlogits = nn.softmax_cross_entropy_backward_fused(1.0 / (n * 10), z, dl)
    else:
        loss, z = nn.softmax_cross_entropy(logits, dl, avoid_overflow=True, reduction="mean")
        dlogits = nn.softmax_cross_entropy_backward(1.0 / (n * 10), z, dl)
    g = {"w3": F.matmul(F.t(dlogits), flat), "b3": F.reshape(F.sum(dlogits, axis=0), -1)}
    dp2 = F.reshape(F.matmul(dlogits, dev["w3"]), *p2.shape)
    da2 = F.mul_(nn.max_pool2d_backward(r2, dp2, 2), m2)
    dp1, g["w2"], g["b2"] = nn.conv2d_backward(p1, dev["w2"], da2)
    da1 = F.mul_(nn.max_pool2d_backward(r1, dp1, 2), m1)
    _, g["w1"], g["b1"] = nn.conv2d_backward(dx, dev["w1"], da1)
    g["b2"], g["b1"] = F.reshape(g["b2"], -1), F.reshape(g["b1"], -1)
    return loss, g


@pytest.mark.parametrize("fused", [True, False])
def test_mnist_cnn_training(gpu, fused):
    """Thirty Adam steps on 256 synthetic digits.  `fused`: unfold and the criterion as one node each
    (what the bypass rules select); otherwise every layer node for node.  The first step's gradients are held
    to the float64 mirror's, the loss of every step too, and the loss must fall."""
    W = gpu
    F = W.functional
    rng = np.random.default_rng(11)
    n = 256
    x, labels = _digits(rng, n)
    params = _params(rng)
    F.ENABLE_SYMBOLIC_PATH = fused
    try:
        dev = {k: F.from_numpy(v) for k, v in params.items()}
        opt = {k: W.optimizers.Adam(dev[k], lr=0.01) for k in dev}
        dx, dl = F.from_numpy(x), F.from_numpy(labels)
        ref = {k: v.astype(np.float64) for k, v in params.items()}
        state = {k: (np.zeros_like(v), np.zeros_like(v)) for k, v in ref.items()}
        x64 = x.astype(np.float64)
        losses = []
        for t in range(1, 31):
            loss, g = _device_step(W, dev, dx, dl, n, fused)
            want_loss, want_g = model_loss_and_grads(ref, x64, labels)
            got = float(loss.numpy().ravel()[0])
            losses.append(got)
            assert abs(got - want_loss) <= 3e-4 * abs(want_loss) + 1e-6, (t, got, want_loss)
            if t == 1:
                for k in want_g:
                    scale = np.max(np.abs(want_g[k]))
                    np.testing.assert_allclose(g[k].numpy().reshape(want_g[k].shape), want_g[k], rtol=0,
                                               atol=2e-5 * scale, err_msg=k)
            for k in dev:
                opt[k].step(g[k])
                m, v = state[k]
                m += (want_g[k] - m) * (1 - 0.9)
                v += (1 - 0.999) * (want_g[k] * want_g[k] - v)
                lr_t = 0.01 * np.sqrt(1 - 0.999 ** t) / (1 - 0.9 ** t)
                ref[k] -= (m * lr_t) / (1e-7 + np.sqrt(v))
        assert losses[-1] < 0.6 * losses[0], losses
    finally:
        F.ENABLE_SYMBOLIC_PATH = True
