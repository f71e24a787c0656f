"""The GPT-2 example's model on the device: its positional embedding node (bit-exact against the
restated reference loop) and the whole forward from token ids to logits against float64."""
import importlib

import numpy as np
import pytest

from helpers import assert_bit_equal

pytestmark = pytest.mark.gpu
f32 = np.float32


@pytest.mark.parametrize("n,t,vocab,n_ctx,dim", [(1, 1, 5, 3, 4), (2, 7, 50, 16, 12), (3, 33, 1000, 64, 70),
                                                 (2, 100, 5000, 128, 768)])
def test_positional_embedding_bits(gpu, O, n, t, vocab, n_ctx, dim):
    W = gpu
    gpt2 = importlib.import_module("cl-waffe2_amd.gpt2")
    rng = np.random.default_rng(n * 100 + t)
    wte = rng.standard_normal((vocab, dim)).astype(f32)
    wpe = rng.standard_normal((n_ctx, dim)).astype(f32)
    ctx = rng.integers(0, vocab, (n, t)).astype(f32)
    want = O.gpt2_positional_embedding(ctx, wte, wpe)
    got = gpt2.positional_embedding(W.HIPTensor.from_numpy(ctx), W.HIPTensor.from_numpy(wte), W.HIPTensor.from_numpy(wpe))
    assert got.shape == [n, t, dim]
    assert_bit_equal(got.numpy(), want, "wte[id] + wpe[position]")


def test_positional_embedding_ids(gpu):
    """Ids are rounded to nearest with ties to even (Common Lisp's ROUND) and clamped to the table."""
    W = gpu
    gpt2 = importlib.import_module("cl-waffe2_amd.gpt2")
    wte = np.arange(10, dtype=f32).reshape(10, 1) * np.ones((1, 4), f32)
    wpe = np.zeros((8, 4), f32)
    ctx = np.array([[0.5, 1.5, 2.5, 3.49, 8.6, 9.0, 42.0, -3.0]], f32)
    got = gpt2.positional_embedding(W.HIPTensor.from_numpy(ctx), W.HIPTensor.from_numpy(wte), W.HIPTensor.from_numpy(wpe))
    assert list(got.numpy()[0, :, 0]) == [0.0, 2.0, 2.0, 3.0, 9.0, 9.0, 9.0, 0.0]
    odd = np.array([[np.nan, np.inf, -np.inf]], f32)
    got = gpt2.positional_embedding(W.HIPTensor.from_numpy(odd), W.HIPTensor.from_numpy(wte), W.HIPTensor.from_numpy(wpe))
    assert list(got.numpy()[0, :, 0]) == [0.0, 9.0, 0.0]
    with pytest.raises(W.HIPError):  # more positions than wpe holds
        gpt2.positional_embedding(W.HIPTensor.from_numpy(np.zeros((1, 9), f32)), W.HIPTensor.from_numpy(wte),
                                  W.HIPTensor.from_numpy(wpe))


@pytest.mark.parametrize("mode", ["fused", "nodes"])
def test_model_forward_small(gpu, mode):
    from oracle import gpt2_block_ref as ref
    W = gpu
    gpt2 = importlib.import_module("cl-waffe2_amd.gpt2")
    cfg = dict(batch=2, seq=24, d_model=64, n_head=4, head_dim=16, d_ff=128, eps=1e-5)
    vocab, n_ctx, layers = 300, 32, 3
    rng = np.random.default_rng(12)
    model = {"wte": (rng.standard_normal((vocab, 64)) * 0.1).astype(f32),
             "wpe": (rng.standard_normal((n_ctx, 64)) * 0.1).astype(f32),
             "ln_f_g": (1 + 0.1 * rng.standard_normal(64)).astype(f32), "ln_f_b": (0.1 * rng.standard_normal(64)).astype(f32),
             "layers": []}
    for i in range(layers):
        p = gpt2.make_block_params(20 + i, cfg)
        for k in p:
            if k.startswith("w_"):
                p[k] = (rng.standard_normal(p[k].shape) * 0.1).astype(f32)
            elif k.startswith("b_") or k.endswith("_b"):
                p[k] = (rng.standard_normal(p[k].shape) * 0.1).astype(f32)
        model["layers"].append(p)
    tokens = rng.integers(0, vocab, (2, 24)).astype(f32)
    want = ref.model_forward(tokens, model, cfg["n_head"], cfg["eps"])
    dev = {k: (W.HIPTensor.from_numpy(v) if k != "layers" else [gpt2.to_device(p) for p in v]) for k, v in model.items()}
    got = gpt2.model_forward(W.HIPTensor.from_numpy(tokens), dev, cfg=cfg, mode=mode).numpy()
    assert got.shape == (2, 24, vocab)
    np.testing.assert_allclose(got, want, rtol=2e-4, atol=2e-4)
    # the next token by !argmax over the last position's logits, as gpt2-inference takes it
    assert np.array_equal(got[:, -1].argmax(-1), want[:, -1].argmax(-1))
