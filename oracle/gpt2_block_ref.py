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
