"""float64 closed form of the GPT-2-small-style block forward (pre-LayerNorm,
causal softmax attention scaled by 1/sqrt(head_dim), tanh-form GELU MLP).

TEST INFRASTRUCTURE ONLY: the checker for the block forward.  The op recipes
follow the reference (LayerNorm-Revisit examples/gpt-2/utils.lisp:114-127, GELU
source/nn/activation.lisp:45-66, weights [in, out] examples/gpt-2/model.lisp:
118-122); the attention definition is the standard one the benchmark
configuration states, because the reference example has no causal mask and
divides by the sequence length (examples/gpt-2/utils.lisp:233-237).
"""
import numpy as np


def layer_norm(x, g, b, eps):
    mu = x.mean(axis=-1, keepdims=True)
    var = ((x - mu) ** 2).mean(axis=-1, keepdims=True)
    return (x - mu) / np.sqrt(var + eps) * g + b


def gelu(x):
    c = x.dtype.type
    return c(0.5) * x * (c(1.0) + np.tanh(c(np.sqrt(2.0 / np.pi)) * (x + c(0.044715) * x ** 3)))


def block_forward(x, p, n_head, eps=1e-5, dtype=np.float64):
    """dtype float64: the checker.  dtype float32: the same recipe in the
    arithmetic of the CPU path, used only to time a CPU baseline."""
    x = x.astype(dtype)
    p = {k: v.astype(dtype) for k, v in p.items()}
    B, T, D = x.shape
    hd = D // n_head
    h = layer_norm(x, p["ln1_g"], p["ln1_b"], eps)
    qkv = h @ p["w_qkv"] + p["b_qkv"]
    q, k, v = (qkv[..., i * D:(i + 1) * D].reshape(B, T, n_head, hd).transpose(0, 2, 1, 3) for i in range(3))
    s = (q @ k.transpose(0, 1, 3, 2)) / dtype(np.sqrt(hd))
    s = np.where(np.tril(np.ones((T, T), bool)), s, dtype(-np.inf))
    e = np.exp(s - s.max(axis=-1, keepdims=True))
    pr = e / e.sum(axis=-1, keepdims=True)
    ctx = (pr @ v).transpose(0, 2, 1, 3).reshape(B, T, D)
    x1 = x + ctx @ p["w_o"] + p["b_o"]
    h2 = layer_norm(x1, p["ln2_g"], p["ln2_b"], eps)
    m = gelu(h2 @ p["w_fc"] + p["b_fc"]) @ p["w_proj"] + p["b_proj"]
    return x1 + m


def block_forward_with_scale(x, p, n_head, eps=1e-5):
    """The float64 block forward and, per output element, the magnitude the last products
    of each residual branch sum over: |x| + |ctx| |W_o| + |gelu(..)| |W_proj| (+ biases).
    An implementation whose products are each within r * sum |a||b| of the exact ones is
    within about r times this of the exact output: the two last products contribute exactly
    that, and what the earlier ones pass on arrives through sums of 768 to 3072 terms of
    either sign and stays well below it (a worst-case propagation, every term aligned, is
    five orders of magnitude above what any arithmetic produces and tests nothing).
    One sequence at a time: the float64 score tensors of all eight would be gigabytes."""
    f8 = np.float64
    P = {k: v.astype(f8) for k, v in p.items()}
    outs, scales = [], []
    for xs in x.astype(f8):
        T, D = xs.shape
        hd = D // n_head
        h = layer_norm(xs, P["ln1_g"], P["ln1_b"], eps)
        qkv = h @ P["w_qkv"] + P["b_qkv"]
        q, k, v = (qkv[:, i * D:(i + 1) * D].reshape(T, n_head, hd).transpose(1, 0, 2) for i in range(3))
        s = (q @ k.transpose(0, 2, 1)) / np.sqrt(hd)
        s = np.where(np.tril(np.ones((T, T), bool)), s, -np.inf)
        e = np.exp(s - s.max(axis=-1, keepdims=True))
        ctx = ((e / e.sum(axis=-1, keepdims=True)) @ v).transpose(1, 0, 2).reshape(T, D)
        x1 = xs + ctx @ P["w_o"] + P["b_o"]
        a = gelu(layer_norm(x1, P["ln2_g"], P["ln2_b"], eps) @ P["w_fc"] + P["b_fc"])
        outs.append(x1 + a @ P["w_proj"] + P["b_proj"])
        scales.append(np.abs(xs) + np.abs(ctx) @ np.abs(P["w_o"]) + np.abs(P["b_o"]) +
                      np.abs(a) @ np.abs(P["w_proj"]) + np.abs(P["b_proj"]))
    return np.stack(outs), np.stack(scales)


def gelu_derivative(x):
    """d/dx of the tanh-form GELU: 0.5 (1 + t) + 0.5 x (1 - t^2) c (1 + 3 a x^2), t = tanh(c (x + a x^3))."""
    c, a = np.sqrt(2.0 / np.pi), 0.044715
    t = np.tanh(c * (x + a * x ** 3))
    return 0.5 * (1.0 + t) + 0.5 * x * (1.0 - t * t) * c * (1.0 + 3.0 * a * x * x)


def layer_norm_backward(x, g, dout, eps):
    """(dx, dgamma, dbeta, |terms| of dx, |terms| of dgamma) of y = (x - u) / sqrt(s + eps) * g + b over the last axis
    (source/nn/norms.lisp:72-82): with xh = (x - u) rstd and dyh = dout g,
    dx = rstd (dyh - mean(dyh) - xh mean(dyh xh))."""
    mu = x.mean(axis=-1, keepdims=True)
    rstd = 1.0 / np.sqrt(((x - mu) ** 2).mean(axis=-1, keepdims=True) + eps)
    xh = (x - mu) * rstd
    dyh = dout * g
    m1 = dyh.mean(axis=-1, keepdims=True)
    m2 = (dyh * xh).mean(axis=-1, keepdims=True)
    dx = rstd * (dyh - m1 - xh * m2)
    mag = rstd * (np.abs(dyh) + np.abs(dyh).mean(axis=-1, keepdims=True) +
                  np.abs(xh) * np.abs(dyh * xh).mean(axis=-1, keepdims=True))
    lead = tuple(range(x.ndim - 1))
    return dx, (dout * xh).sum(axis=lead), dout.sum(axis=lead), mag, np.abs(dout * xh).sum(axis=lead)


def block_backward(x, p, n_head, dout, eps=1e-5):
    """Gradients of sum(block_forward(x, p) * dout) in float64, derived by hand from the forward above
    (pinned by central differences in tests/test_oracle_block_backward.py).  Returns (grads, scales):
    `grads` maps 'x' and every parameter name to its gradient; `scales` maps the same names to the
    magnitude the last product or sum that forms that gradient adds up (sum |a||b|), the yardstick
    an fp32 implementation's error is held against.  One sequence at a time."""
    f8 = np.float64
    P = {k: v.astype(f8) for k, v in p.items()}
    D = x.shape[-1]
    hd = D // n_head
    sc = 1.0 / np.sqrt(hd)
    grads = {k: np.zeros_like(v) for k, v in P.items()}
    scales = {k: np.zeros_like(v) for k, v in P.items()}
    dxs, sxs = [], []
    for xs, do in zip(x.astype(f8), dout.astype(f8)):
        T = xs.shape[0]
        # forward, keeping what the backward reads
        h = layer_norm(xs, P["ln1_g"], P["ln1_b"], eps)
        qkv = h @ P["w_qkv"] + P["b_qkv"]
        q, k, v = (qkv[:, i * D:(i + 1) * D].reshape(T, n_head, hd).transpose(1, 0, 2) for i in range(3))
        s = (q @ k.transpose(0, 2, 1)) * sc
        s = np.where(np.tril(np.ones((T, T), bool)), s, -np.inf)
        e = np.exp(s - s.max(axis=-1, keepdims=True))
        pr = e / e.sum(axis=-1, keepdims=True)
        ctx = (pr @ v).transpose(1, 0, 2).reshape(T, D)
        x1 = xs + ctx @ P["w_o"] + P["b_o"]
        h2 = layer_norm(x1, P["ln2_g"], P["ln2_b"], eps)
        z = h2 @ P["w_fc"] + P["b_fc"]
        f = gelu(z)

        def acc(name, g, s_):
            grads[name] += g
            scales[name] += s_

        # out = x1 + f w_proj + b_proj
        acc("w_proj", f.T @ do, np.abs(f).T @ np.abs(do))
        acc("b_proj", do.sum(axis=0), np.abs(do).sum(axis=0))
        df = do @ P["w_proj"].T
        dz = df * gelu_derivative(z)
        acc("w_fc", h2.T @ dz, np.abs(h2).T @ np.abs(dz))
        acc("b_fc", dz.sum(axis=0), np.abs(dz).sum(axis=0))
        dh2 = dz @ P["w_fc"].T
        dln2, dg2, db2, mag2, mag_g2 = layer_norm_backward(x1, P["ln2_g"], dh2, eps)
        acc("ln2_g", dg2, mag_g2)
        acc("ln2_b", db2, np.abs(dh2).sum(axis=0))
        dx1 = do + dln2
        # x1 = x + ctx w_o + b_o
        acc("w_o", ctx.T @ dx1, np.abs(ctx).T @ np.abs(dx1))
        acc("b_o", dx1.sum(axis=0), np.abs(dx1).sum(axis=0))
        dctx = (dx1 @ P["w_o"].T).reshape(T, n_head, hd).transpose(1, 0, 2)
        # ctx = softmax(scale q k^T + mask) v
        dv = pr.transpose(0, 2, 1) @ dctx
        dp = dctx @ v.transpose(0, 2, 1)
        ds = pr * (dp - (dp * pr).sum(axis=-1, keepdims=True))
        dq = (ds @ k) * sc
        dk = (ds.transpose(0, 2, 1) @ q) * sc
        dqkv = np.concatenate([t.transpose(1, 0, 2).reshape(T, D) for t in (dq, dk, dv)], axis=1)
        acc("w_qkv", h.T @ dqkv, np.abs(h).T @ np.abs(dqkv))
        acc("b_qkv", dqkv.sum(axis=0), np.abs(dqkv).sum(axis=0))
        dh = dqkv @ P["w_qkv"].T
        dln1, dg1, db1, mag1, mag_g1 = layer_norm_backward(xs, P["ln1_g"], dh, eps)
        acc("ln1_g", dg1, mag_g1)
        acc("ln1_b", db1, np.abs(dh).sum(axis=0))
        dxs.append(dx1 + dln1)
        sxs.append(np.abs(do) + mag2 + mag1)
    grads["x"] = np.stack(dxs)
    scales["x"] = np.stack(sxs)
    return grads, scales


def model_forward(tokens, model, n_head, eps=1e-5):
    """float64 closed form of the example's GPT2 model with the benchmark's attention in the layers
    (examples/gpt-2/model.lisp:137-196): wte[token] + wpe[position], the blocks, the final LayerNorm,
    logits = x . wte^T."""
    f8 = np.float64
    ids = np.rint(np.asarray(tokens)).astype(np.int64)
    x = model["wte"].astype(f8)[ids] + model["wpe"].astype(f8)[np.arange(ids.shape[1])][None]
    for layer in model["layers"]:
        x = block_forward(x, layer, n_head, eps)
    x = layer_norm(x, model["ln_f_g"].astype(f8), model["ln_f_b"].astype(f8), eps)
    return x @ model["wte"].astype(f8).T
