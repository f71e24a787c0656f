"""MatMulNode at the shapes of the GPT-2-small block (benchmark configuration 5) against
float64, held to the bar stated for products: |c - exact| <= 1e-5 * sum_k |a||b| per
element.  The tile shape, the streaming or register-staged kernel and the split over K
are all chosen from the shape, so the shapes themselves have to be tested: the three
projections in both layouts of the right operand, the weight gradient that splits K, and
the 96 batched products of attention read in place from the fused projection.  float64
truth on a fixed sample of output rows (every 29th, plus the first and last tile rows)."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

REL = 1e-5


def _rows(m):
    rows = sorted(set(range(0, m, 29)) | set(range(0, 130)) | set(range(m - 130, m)))
    return np.array([r for r in rows if 0 <= r < m])


def _check(got, A64, B64, rows, what):
    want = A64[rows] @ B64
    scale = np.abs(A64[rows]) @ np.abs(B64)
    ratio = np.abs(got[rows].astype(np.float64) - want) / scale
    print(what, "rows checked", len(rows), "worst error / sum |a||b|:", ratio.max(), flush=True)
    assert ratio.max() <= REL, (what, ratio.max())


@pytest.mark.parametrize("m, n, k", [(8192, 2304, 768), (8192, 768, 768), (8192, 3072, 768), (8192, 768, 3072)])
@pytest.mark.parametrize("right_stored_transposed", [False, True])
def test_projection_shapes(gpu, m, n, k, right_stored_transposed):
    F = gpu.functional
    rng = np.random.Generator(np.random.PCG64(5))
    A = rng.standard_normal((m, k)).astype(np.float32)
    B = (rng.standard_normal((k, n)) * 0.02).astype(np.float32)
    dA = F.from_numpy(A)
    dB = F.t(F.from_numpy(np.ascontiguousarray(B.T))) if right_stored_transposed else F.from_numpy(B)
    got = F.matmul(dA, dB).numpy()
    assert got.shape == (m, n) and np.isfinite(got).all()
    rows = _rows(m)
    assert len(rows) >= 256
    _check(got, A.astype(np.float64), B.astype(np.float64), rows, f"{m}x{n}x{k} right^T={right_stored_transposed}")


def test_weight_gradient_split_over_k(gpu):
    """dW = x^T . dY, (768 x 8192) . (8192 x 3072): few output tiles and a long K, which the
    library splits over K; the left operand is stored (8192, 768)."""
    F = gpu.functional
    rng = np.random.Generator(np.random.PCG64(6))
    X = rng.standard_normal((8192, 768)).astype(np.float32)
    dY = rng.standard_normal((8192, 3072)).astype(np.float32)
    got = F.matmul(F.t(F.from_numpy(X)), F.from_numpy(dY)).numpy()
    assert got.shape == (768, 3072)
    rows = _rows(768)
    _check(got, X.T.astype(np.float64), dY.astype(np.float64), rows, "768x3072x8192 split over K")


def test_attention_products_read_in_place(gpu):
    """The 96 score products (1024 x 64) . (64 x 1024) and the 96 context products
    (1024 x 1024) . (1024 x 64) of B 8, H 12, with q, k, v as (B, H, T, 64) views of the
    (B, T, 3, H, 64) projection (no copies), every batch checked on sampled rows."""
    W = gpu
    F = W.functional
    rng = np.random.Generator(np.random.PCG64(7))
    B, T, H, hd = 8, 1024, 12, 64
    qkv = rng.standard_normal((B, T, 3, H, hd)).astype(np.float32)
    d = F.from_numpy(qkv)
    # (B, 1, H, T, hd) strided windows of the projection, as the block forward takes them
    q, k, v = (d.view(True, True, i, True, True).permute(0, 2, 3, 1, 4) for i in range(3))
    s = F.matmul(q, F.t(k)).numpy().reshape(B, H, T, T)
    rows = np.arange(0, T, 7)
    q64, k64, v64 = (qkv[:, :, i].transpose(0, 2, 1, 3).astype(np.float64) for i in range(3))
    worst = 0.0
    for b in range(B):
        for h in range(H):
            want = q64[b, h][rows] @ k64[b, h].T
            scale = np.abs(q64[b, h][rows]) @ np.abs(k64[b, h].T)
            worst = max(worst, (np.abs(s[b, h][rows] - want) / scale).max())
    print("scores worst error / sum |a||b|:", worst, flush=True)
    assert worst <= REL
    p = np.abs(rng.standard_normal((B, H, T, T))).astype(np.float32)
    p /= p.sum(axis=-1, keepdims=True)
    ctx = F.matmul(F.from_numpy(p.reshape(B, 1, H, T, T)), v).numpy().reshape(B, H, T, hd)
    worst = 0.0
    for b in range(B):
        for h in range(H):
            want = p[b, h][rows].astype(np.float64) @ v64[b, h]
            scale = np.abs(p[b, h][rows]).astype(np.float64) @ np.abs(v64[b, h])
            worst = max(worst, (np.abs(ctx[b, h][rows] - want) / scale).max())
    print("context worst error / sum |a||b|:", worst, flush=True)
    assert worst <= REL
