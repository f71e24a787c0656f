"""wf2hip_attention_f32 against the float64 closed form.

The kernel replaces the !matmul / scale / mask / !softmax / !matmul chain of
the reference's SelfAttention (examples/gpt-2/utils.lisp:222-243).  The
reference has no vectors for it (its example runs without mask and divides by
the sequence length), so the contract is the textbook definition evaluated in
float64: **parity unpinned by the reference**.  Bar: 1e-5 of max |V| absolute
(outputs are convex combinations of V rows; binary32 products of 64 terms and
sums of up to `seq` terms sit well inside it).
"""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def reference(q, k, v, scale, causal):
    q, k, v = (a.astype(np.float64) for a in (q, k, v))
    s = np.einsum("bhid,bhjd->bhij", q, k) * scale
    if causal:
        T = q.shape[2]
        s = np.where(np.tril(np.ones((T, T), bool)), s, -np.inf)
    s = s - s.max(axis=-1, keepdims=True)
    p = np.exp(s)
    p /= p.sum(axis=-1, keepdims=True)
    return np.einsum("bhij,bhjd->bhid", p, v)


def check(got, want, v):
    err = np.abs(got.astype(np.float64) - want).max()
    assert err <= 1e-5 * np.abs(v).max(), err


@pytest.mark.parametrize("B,H,T", [(1, 1, 1), (1, 2, 31), (2, 3, 64), (1, 2, 65), (2, 2, 128),
                                   (1, 3, 200), (2, 2, 257), (1, 2, 1024)])
@pytest.mark.parametrize("causal", [True, False])
def test_attention_contiguous(gpu, B, H, T, causal):
    W = gpu
    F = W.functional
    rng = np.random.default_rng(1000 * T + B + H + causal)
    q, k, v = (rng.standard_normal((B, H, T, 64)).astype(np.float32) for _ in range(3))
    q *= 2.0  # scores of a few units: a peaked softmax
    out = F.attention(F.from_numpy(q), F.from_numpy(k), F.from_numpy(v), causal=causal)
    check(out.numpy(), reference(q, k, v, 0.125, causal), v)


@pytest.mark.parametrize("hd", [4, 12, 32, 60])
def test_attention_narrow_heads(gpu, hd):
    W = gpu
    F = W.functional
    rng = np.random.default_rng(hd)
    q, k, v = (rng.standard_normal((2, 2, 100, hd)).astype(np.float32) for _ in range(3))
    out = F.attention(F.from_numpy(q), F.from_numpy(k), F.from_numpy(v), causal=True)
    check(out.numpy(), reference(q, k, v, 1.0 / np.sqrt(hd), True), v)


def test_attention_heads_in_place(gpu):
    """q/k/v read through strides from one (B, T, 3, H, 64) projection buffer,
    context written as (B, T, H*64): the layout of the block forward."""
    W = gpu
    F = W.functional
    B, T, H = 2, 192, 3
    rng = np.random.default_rng(7)
    qkv = rng.standard_normal((B, T, 3 * H, 64)).astype(np.float32)
    d = F.from_numpy(qkv)
    q, k, v = (d.view(True, True, (i * H, (i + 1) * H), True).permute(0, 2, 1, 3) for i in range(3))
    store = W.HIPTensor([B, T, H, 64])
    F.attention(q, k, v, out=store.permute(0, 2, 1, 3), scale=0.2, causal=True)
    hq, hk, hv = (qkv[:, :, i * H:(i + 1) * H].transpose(0, 2, 1, 3) for i in range(3))
    want = reference(hq, hk, hv, 0.2, True).transpose(0, 2, 1, 3)
    check(store.numpy(), want, hv)


def test_attention_properties_full_size(gpu):
    """(8, 12, 1024, 64), the benchmark's shape: rows of a causal result depend
    only on earlier positions (a change to the last key/value leaves all earlier
    rows bit-identical), position 0 returns V[0], and constant V is reproduced."""
    W = gpu
    F = W.functional
    B, H, T = 8, 12, 1024
    rng = np.random.default_rng(11)
    q, k, v = (rng.standard_normal((B, H, T, 64)).astype(np.float32) for _ in range(3))
    dq, dk, dv = F.from_numpy(q), F.from_numpy(k), F.from_numpy(v)
    base = F.attention(dq, dk, dv, causal=True).numpy()
    np.testing.assert_allclose(base[:, :, 0], v[:, :, 0], rtol=1e-6, atol=0)
    k2, v2 = k.copy(), v.copy()
    k2[:, :, -1] += 1.0
    v2[:, :, -1] -= 3.0
    moved = F.attention(dq, F.from_numpy(k2), F.from_numpy(v2), causal=True).numpy()
    assert np.array_equal(base[:, :, :-1].view(np.uint32), moved[:, :, :-1].view(np.uint32))
    assert not np.array_equal(base[:, :, -1], moved[:, :, -1])
    const = np.broadcast_to(np.float32(0.75), v.shape).copy()
    got = F.attention(dq, dk, F.from_numpy(const), causal=False).numpy()
    np.testing.assert_allclose(got, 0.75, rtol=1e-5)
    # one (batch, head) slice against float64
    want = reference(q[3:4, 5:6], k[3:4, 5:6], v[3:4, 5:6], 0.125, True)
    check(base[3:4, 5:6], want, v)


def test_attention_argument_checks(gpu):
    W = gpu
    F = W.functional
    lib = W.lib.get()
    a = W.HIPTensor([1, 1, 8, 64])
    d = W.lib.AttentionDesc()
    d.batch, d.heads, d.seq, d.head_dim = 1, 1, 8, 128
    for f in (d.q_stride, d.k_stride, d.v_stride, d.o_stride):
        f[0], f[1], f[2] = 512, 512, 64
    d.scale = 1.0
    p = C.c_void_p(a.ptr)
    o = W.HIPTensor([1, 1, 8, 64])
    assert lib.wf2hip_attention_f32(C.byref(d), p, p, p, C.c_void_p(o.ptr)) == -4   # head_dim
    d.head_dim = 64
    assert lib.wf2hip_attention_f32(C.byref(d), p, p, p, p) == W.lib.EOVERLAP
    d.q_stride[2] = 66
    assert lib.wf2hip_attention_f32(C.byref(d), p, p, p, C.c_void_p(o.ptr)) == -1
    d.q_stride[2] = 64
    assert lib.wf2hip_attention_f32(C.byref(d), p, p, p, C.c_void_p(o.ptr)) == 0
    d.seq = 0
    assert lib.wf2hip_attention_f32(C.byref(d), p, p, p, C.c_void_p(o.ptr)) == 0
    with pytest.raises(ValueError):
        F.attention(a, a, W.HIPTensor([1, 1, 4, 64]))
