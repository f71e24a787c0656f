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
