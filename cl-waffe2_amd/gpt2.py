"""GPT-2-small-style transformer block forward on HIPTensor nodes.

Op decomposition follows the reference's GPT-2 example
(``examples/gpt-2/model.lisp:95-137`` block wiring, ``utils.lisp:114-127``
LayerNorm-Revisit, ``:204-239`` split-heads / SelfAttention / merge-heads,
``source/nn/activation.lisp:45-66`` GELU) with the standard definitions the
benchmark configuration asks for where the example deviates: causal mask,
scores scaled by 1/sqrt(head_dim), softmax over the key axis, max-subtracted.
Weights are stored ``[in, out]`` and applied as ``x @ W + b`` like the example
(``model.lisp:118-122``).

Two modes:

``nodes``  every step is one of the backend's AbstractNode implementations:
           LayerNorm and GELU node for node, heads materialised with
           MoveTensorNode copies of sliced/permuted views, scaling and masking
           as MulNode / AddNode with broadcast operands, row softmax kernel.
``fused``  the same mathematics with fused kernels: LayerNorm in one pass,
           bias / GELU / residual in the gemm epilogues, and causal attention
           as a single kernel that reads q/k/v straight out of the
           (B, T, 3, H, hd) projection through strides, never materialises the
           (B, H, T, T) scores and writes the context straight into
           (B, T, H*hd).
``fused_matmul_attention``  as ``fused`` but attention built from two batched
           products with causal tile skipping and the fused scale+mask+softmax
           row kernel (scores materialised once).
"""
from __future__ import annotations

import ctypes as C
import math

import numpy as np

from . import functional as F
from . import lib as _lib
from .tensor import HIPTensor

CONFIG = dict(batch=8, seq=1024, d_model=768, n_head=12, head_dim=64, d_ff=3072, eps=1e-5)


def make_block_params(seed: int = 5, cfg: dict = CONFIG) -> dict:
    """Weights ~ N(0, 0.02^2), zero biases, LayerNorm gamma 1 / beta 0; drawn
    after the input from one PCG64 stream (see make_block_input)."""
    rng = np.random.Generator(np.random.PCG64(seed))
    d, ff = cfg["d_model"], cfg["d_ff"]
    rng.standard_normal((cfg["batch"], cfg["seq"], d))  # the input comes first
    w = lambda *s: (rng.standard_normal(s) * 0.02).astype(np.float32)  # noqa: E731
    return {
        "w_qkv": w(d, 3 * d), "w_o": w(d, d), "w_fc": w(d, ff), "w_proj": w(ff, d),
        "b_qkv": np.zeros(3 * d, np.float32), "b_o": np.zeros(d, np.float32),
        "b_fc": np.zeros(ff, np.float32), "b_proj": np.zeros(d, np.float32),
        "ln1_g": np.ones(d, np.float32), "ln1_b": np.zeros(d, np.float32),
        "ln2_g": np.ones(d, np.float32), "ln2_b": np.zeros(d, np.float32),
    }


def make_block_input(seed: int = 5, cfg: dict = CONFIG) -> np.ndarray:
    rng = np.random.Generator(np.random.PCG64(seed))
    return rng.standard_normal((cfg["batch"], cfg["seq"], cfg["d_model"])).astype(np.float32)


def to_device(params: dict) -> dict:
    return {k: HIPTensor.from_numpy(v) for k, v in params.items()}


def causal_mask(seq: int) -> HIPTensor:
    """(1, 1, T, T) additive mask: 0 on and below the diagonal, -inf above."""
    m = np.where(np.tril(np.ones((seq, seq), bool)), 0.0, -np.inf).astype(np.float32)
    return HIPTensor.from_numpy(m.reshape(1, 1, seq, seq))


def _linear(x: HIPTensor, w: HIPTensor, b: HIPTensor) -> HIPTensor:
    """``(!add (!matmul x w) (%transform b[i] -> [~ i]))``; the product is a
    fresh tensor, so the bias is added in place."""
    return F.add_(F.matmul(x, w), b)


def block_forward(x: HIPTensor, p: dict, mode: str = "fused", cfg: dict = CONFIG,
                  mask: HIPTensor | None = None, saved: dict | None = None) -> HIPTensor:
    """`saved`, when given (mode 'fused' only), receives what the fused nodes keep for their
    backward (their inputs: ``:save-for-backward-names`` of the Lisp nodes) for `block_backward`."""
    B, T, D = x.shape
    H = cfg["n_head"]
    hd = D // H
    scale = 1.0 / math.sqrt(hd)
    eps = cfg["eps"]
    fused = mode in ("fused", "fused_matmul_attention")
    if mode not in ("fused", "fused_matmul_attention", "nodes"):
        raise ValueError("mode must be 'fused', 'fused_matmul_attention' or 'nodes'")
    ln = F.layer_norm_fused if fused else F.layer_norm
    act = F.gelu_fused if fused else F.gelu

    h = ln(x, p["ln1_g"], p["ln1_b"], eps)
    if fused:
        qkv = F.linear(h, p["w_qkv"], p["b_qkv"])                  # (B, T, 3D), HIP-Linear-Node
    else:
        qkv = _linear(h, p["w_qkv"], p["b_qkv"])

    if mode == "fused" and (hd % 4 != 0 or hd > 64):
        mode = "fused_matmul_attention"   # the attention kernel is built for heads up to 64 wide
    if mode == "fused":
        four = F.reshape(qkv, B, T, 3 * H, hd)
        # (B, H, T, hd) strided windows of the projection, no copy; the context is
        # written straight into its merged (B, T, H*hd) layout
        q, k, v = (four.view(True, True, (i * H, (i + 1) * H), True).permute(0, 2, 1, 3)
                   for i in range(3))
        ctx_store = HIPTensor([B, T, H, hd], initial_element=None)
        # training: the row statistics the attention node's backward reads
        lse = HIPTensor([B, H, T], initial_element=None) if saved is not None else None
        F.attention(q, k, v, out=ctx_store.permute(0, 2, 1, 3), scale=scale, causal=True, lse=lse)
        ctx = F.reshape(ctx_store, B, T, D)
        if saved is not None:
            saved["lse"] = lse
    elif fused:
        five = F.reshape(qkv, B, T, 3, H, hd)
        # (B, 1, H, T, hd) strided windows of the projection, no copy
        q, k, v = (five.view(True, True, i, True, True).permute(0, 2, 3, 1, 4) for i in range(3))
        scores = F.matmul(q, F.t(k), causal=1)                      # (B, 1, H, T, T), lower triangle
        probs = F.causal_softmax_fused(scores, scale)              # HIP-Causal-Softmax-Node
        ctx_store = HIPTensor([B, T, 1, H, hd], initial_element=None)
        F.matmul(probs, v, out=ctx_store.permute(0, 2, 3, 1, 4), causal=2)  # written as (B, T, H*hd)
        ctx = F.reshape(ctx_store, B, T, D)
    else:
        def heads(i):  # split-heads: slice, reshape, permute, materialise
            part = qkv.view(True, True, (i * D, (i + 1) * D))
            return F.copy(F.reshape(part, B, T, H, hd).permute(0, 2, 1, 3))  # (B, H, T, hd)
        q, k, v = heads(0), heads(1), heads(2)
        scores = F.mul_(F.matmul(q, F.t(k)), scale)                 # (B, H, T, T)
        if mask is None:
            mask = causal_mask(T)
        F.add_(scores, mask)                                        # broadcast over (B, H)
        probs = F.softmax_fused(scores)
        ctx = F.matmul(probs, v)                                    # (B, H, T, hd)
        ctx = F.reshape(ctx.permute(0, 2, 1, 3), B, T, D)           # merge-heads (copies)

    if fused:
        # bias, GELU and the residual adds ride in the products' epilogues
        # (HIP-Linear-Residual-Node, HIP-Linear-Node :gelu, HIP-Linear-Residual-Node)
        x1 = F.linear(ctx, p["w_o"], p["b_o"], residual=x)
        h2 = ln(x1, p["ln2_g"], p["ln2_b"], eps)
        if saved is None:
            f = F.linear(h2, p["w_fc"], p["b_fc"], activation="gelu")
        else:
            # the training form: (!gelu-hip (!linear-hip h2 w b)) keeps the pre-activation as the
            # activation node's saved input (one more pass of 12 B per element forward) where the
            # :gelu epilogue would recompute it by a whole product backward
            if mode != "fused":
                raise ValueError("block_forward: saved tensors are kept for mode 'fused'")
            z = F.linear(h2, p["w_fc"], p["b_fc"])
            f = F.gelu_fused(z)
            saved.update(x=x, h=h, qkv=qkv, ctx=ctx, x1=x1, h2=h2, z=z, f=f)
        return F.linear(f, p["w_proj"], p["b_proj"], residual=x1)
    attn = _linear(ctx, p["w_o"], p["b_o"])
    x1 = F.add(x, attn)                                             # residual
    h2 = ln(x1, p["ln2_g"], p["ln2_b"], eps)
    f = act(_linear(h2, p["w_fc"], p["b_fc"]))
    m = _linear(f, p["w_proj"], p["b_proj"])
    return F.add_(m, x1)                                            # residual, in place in m


def block_backward(dout: HIPTensor, saved: dict, p: dict, cfg: dict = CONFIG):
    """Gradients of the fused block from what `block_forward(..., saved=...)` kept: every fused
    node's backward in reverse order, composed as the Lisp nodes compose theirs (HIP-Linear-Node,
    HIP-Linear-Residual-Node, HIP-LayerNorm-Node, HIP-Attention-Node with the probabilities
    recomputed), the gradient adders of the two residual forks as AddNodes.  Returns (dx, grads)
    with `grads` keyed like the parameters."""
    x, h, qkv, ctx, x1, h2, z, f = (saved[k] for k in ("x", "h", "qkv", "ctx", "x1", "h2", "z", "f"))
    B, T, D = x.shape
    H = cfg["n_head"]
    hd = D // H
    eps = cfg["eps"]
    g = {}
    # out = f . w_proj + b_proj + x1
    df, g["w_proj"], g["b_proj"] = F.linear_backward(f, p["w_proj"], p["b_proj"], dout)
    # f = gelu(z), z = h2 . w_fc + b_fc  (HIP-Activation-Node on HIP-Linear-Node; df is not needed again)
    dz = F.activation_backward("gelu", z, df, in_place=True)
    dh2, g["w_fc"], g["b_fc"] = F.linear_backward(h2, p["w_fc"], p["b_fc"], dz)
    # h2 = LayerNorm(x1); x1 also feeds the residual
    dln2, g["ln2_g"], g["ln2_b"] = F.layer_norm_backward(x1, p["ln2_g"], dh2, eps)
    dx1 = F.add_(dln2, dout)
    # x1 = ctx . w_o + b_o + x
    dctx, g["w_o"], g["b_o"] = F.linear_backward(ctx, p["w_o"], p["b_o"], dx1)
    # ctx = attention(q, k, v), heads read in place from the projection, their gradients
    # written in place into the projection's gradient
    four = F.reshape(qkv, B, T, 3 * H, hd)
    q, k, v = (four.view(True, True, (i * H, (i + 1) * H), True).permute(0, 2, 1, 3) for i in range(3))
    dqkv = HIPTensor([B, T, 3 * H, hd], initial_element=None)
    dq, dk, dv = (dqkv.view(True, True, (i * H, (i + 1) * H), True).permute(0, 2, 1, 3) for i in range(3))
    dctx_heads = F.reshape(dctx, B, T, H, hd).permute(0, 2, 1, 3)
    # with the forward's row statistics: one node, no (B, H, T, T) tensor; without them (heads the
    # attention kernel does not take): the composition with the probabilities recomputed
    F.attention_backward(q, k, v, dctx_heads, scale=1.0 / math.sqrt(hd), causal=True, dq=dq, dk=dk, dv=dv,
                         out=F.reshape(ctx, B, T, H, hd).permute(0, 2, 1, 3) if "lse" in saved else None,
                         lse=saved.get("lse"))
    # qkv = h . w_qkv + b_qkv
    dh, g["w_qkv"], g["b_qkv"] = F.linear_backward(h, p["w_qkv"], p["b_qkv"], F.reshape(dqkv, B, T, 3 * D))
    # h = LayerNorm(x); x also feeds the residual
    dln1, g["ln1_g"], g["ln1_b"] = F.layer_norm_backward(x, p["ln1_g"], dh, eps)
    return F.add_(dln1, dx1), g


def positional_embedding(ctx: HIPTensor, wte: HIPTensor, wpe: HIPTensor) -> HIPTensor:
    """``(call (GPT2PositionalEmbedding ...) ctx wte wpe out)``: token ids (as :float, N x T) to
    wte[id] + wpe[position], (N, T, embedding-size) (``examples/gpt-2/utils.lisp:68-110``)."""
    from . import nodes
    n, t = ctx.shape
    out = HIPTensor([n, t, wte.shape[1]], initial_element=None)
    return nodes.forward("GPT2PositionalEmbedding", ctx, wte, wpe, out)


def model_forward(tokens: HIPTensor, model: dict, cfg: dict = CONFIG, mode: str = "fused") -> HIPTensor:
    """The GPT2 model of the example (``examples/gpt-2/model.lisp:137-196``): positional embedding,
    the layers, the final LayerNorm and the language-model head ``x . wte^T`` (``lm-head``), with the
    benchmark's standard attention in the layers.  `model` holds 'wte', 'wpe', 'ln_f_g', 'ln_f_b' and
    'layers', a list of block parameter dicts.  Returns the logits (N, T, vocab)."""
    x = positional_embedding(tokens, model["wte"], model["wpe"])
    for layer in model["layers"]:
        x = block_forward(x, layer, mode=mode, cfg=cfg)
    ln = F.layer_norm_fused if mode != "nodes" else F.layer_norm
    x = ln(x, model["ln_f_g"], model["ln_f_b"], cfg["eps"])
    return F.matmul(x, F.t(model["wte"]))
