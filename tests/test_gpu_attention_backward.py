"""HIP-Attention-Node-backward (three launches, no (seq, seq) tensor) against float64."""
import importlib

import numpy as np
import pytest

pytestmark = pytest.mark.gpu
f32 = np.float32


def _truth(q, k, v, do, scale, causal):
    Q, K, V, DO = (a.astype(np.float64) for a in (q, k, v, do))
    T = q.shape[2]
    s = Q @ K.transpose(0, 1, 3, 2) * scale
    if causal:
        s = np.where(np.tril(np.ones((T, T), bool)), s, -np.inf)
    e = np.exp(s - s.max(-1, keepdims=True))
    p = e / e.sum(-1, keepdims=True)
    o = p @ V
    dv = p.transpose(0, 1, 3, 2) @ DO
    dp = DO @ V.transpose(0, 1, 3, 2)
    ds = p * (dp - (dp * p).sum(-1, keepdims=True))
    dq, dk = ds @ K * scale, ds.transpose(0, 1, 3, 2) @ Q * scale
    # the magnitude of dS before its two terms cancel: P (|dP| + |D|)
    big = p * (np.abs(dp) + np.abs((dp * p).sum(-1, keepdims=True)))
    mags = (big @ np.abs(K) * scale, big.transpose(0, 1, 3, 2) @ np.abs(Q) * scale,
            p.transpose(0, 1, 3, 2) @ np.abs(DO))
    return o, (dq, dk, dv), mags


@pytest.mark.parametrize("B,H,T,hd,causal", [
    (1, 1, 32, 64, False), (1, 1, 64, 64, True), (1, 2, 128, 64, True), (2, 3, 70, 16, False), (2, 3, 70, 16, True),
    (1, 2, 129, 64, True), (1, 2, 200, 32, True), (2, 2, 257, 64, False), (1, 3, 300, 12, True),
    (1, 2, 512, 64, True), (1, 1, 1024, 64, True), (1, 1, 1000, 64, False)])
def test_attention_backward_kernel(gpu, B, H, T, hd, causal):
    W = gpu
    F = W.functional
    print(f"case B={B} H={H} T={T} hd={hd} causal={causal}", flush=True)
    rng = np.random.default_rng(B * 1000 + T + hd)
    q, k, v, do = (rng.standard_normal((B, H, T, hd)).astype(f32) for _ in range(4))
    scale = 1.0 / np.sqrt(hd)
    o_want, grads, mags = _truth(q, k, v, do, scale, causal)
    tq, tk, tv, tdo = (F.from_numpy(a) for a in (q, k, v, do))
    lse = W.HIPTensor([B, H, T], initial_element=None)
    out = F.attention(tq, tk, tv, causal=causal, lse=lse)
    assert np.max(np.abs(out.numpy() - o_want)) <= 2e-5 * np.abs(v).max()
    # the statistics: log2 of the row sums of exp2(scale log2e q.k)
    s = (q.astype(np.float64) @ k.astype(np.float64).transpose(0, 1, 3, 2)) * scale
    if causal:
        s = np.where(np.tril(np.ones((T, T), bool)), s, -np.inf)
    lse_want = (s.max(-1) + np.log(np.exp(s - s.max(-1, keepdims=True)).sum(-1))) / np.log(2.0)
    assert np.max(np.abs(lse.numpy() - lse_want)) <= 1e-4
    gq, gk, gv = F.attention_backward(tq, tk, tv, tdo, causal=causal, out=out, lse=lse)
    for name, got, want, mag in zip(("dq", "dk", "dv"), (gq, gk, gv), grads, mags):
        ratio = np.abs(got.numpy() - want) / np.maximum(mag, 1e-30)
        print(name, "worst error / magnitude", ratio.max(), flush=True)
        assert ratio.max() <= 1e-5, (name, ratio.max())


def test_attention_backward_on_windows_of_a_projection(gpu):
    """q, k, v read in place from a (B, T, 3H, hd) projection, the gradients written in place into
    the projection's gradient, dout and out laid out (B, T, H, hd): the block's own call.  Then the
    same operands with a contiguous dout, which takes the copying route; both against float64."""
    W = gpu
    F = W.functional
    B, T, H, hd = 2, 150, 3, 32
    rng = np.random.default_rng(4)
    qkv = rng.standard_normal((B, T, 3 * H, hd)).astype(f32)
    do = rng.standard_normal((B, T, H, hd)).astype(f32)
    q, k, v = (np.ascontiguousarray(qkv[:, :, i * H:(i + 1) * H].transpose(0, 2, 1, 3)) for i in range(3))
    scale = 1.0 / np.sqrt(hd)
    _, grads, mags = _truth(q, k, v, np.ascontiguousarray(do.transpose(0, 2, 1, 3)), scale, True)
    t = F.from_numpy(qkv)
    tq, tk, tv = (t.view(True, True, (i * H, (i + 1) * H), True).permute(0, 2, 1, 3) for i in range(3))
    store = W.HIPTensor([B, T, H, hd], initial_element=None)
    lse = W.HIPTensor([B, H, T], initial_element=None)
    out = F.attention(tq, tk, tv, out=store.permute(0, 2, 1, 3), causal=True, lse=lse)
    for contiguous_dout in (False, True):
        dqkv = F.from_numpy(np.full(qkv.shape, np.nan, f32))
        gq, gk, gv = (dqkv.view(True, True, (i * H, (i + 1) * H), True).permute(0, 2, 1, 3) for i in range(3))
        tdo = F.from_numpy(do).permute(0, 2, 1, 3)
        if contiguous_dout:
            tdo = F.copy(tdo)
        F.attention_backward(tq, tk, tv, tdo, causal=True, dq=gq, dk=gk, dv=gv, out=out, lse=lse)
        got = dqkv.numpy()
        assert np.all(np.isfinite(got))
        for i, (want, mag) in enumerate(zip(grads, mags)):
            g = got[:, :, i * H:(i + 1) * H].transpose(0, 2, 1, 3)
            assert np.max(np.abs(g - want) / np.maximum(mag, 1e-30)) <= 1e-5, (contiguous_dout, i)


def test_attention_backward_argument_checks(gpu):
    import ctypes as C
    W = gpu
    F = W.functional
    B, H, T, hd = 1, 1, 16, 8
    x = [F.from_numpy(np.ones((B, H, T, hd), f32)) for _ in range(8)]
    lse = W.HIPTensor([B, H, T])
    d = W.lib.AttentionDesc()
    d.batch, d.heads, d.seq, d.head_dim = B, H, T, hd
    for field in (d.q_stride, d.k_stride, d.v_stride, d.o_stride):
        field[0], field[1], field[2] = H * T * hd, T * hd, hd
    d.scale, d.causal = 1.0, 0
    p = lambda t: C.c_void_p(t.ptr)  # noqa: E731
    lib = W.lib.get()
    ok = lib.wf2hip_attention_backward_f32(C.byref(d), p(x[0]), p(x[1]), p(x[2]), p(x[3]), p(x[4]), p(lse), p(x[5]),
                                           p(x[6]), p(x[7]))
    assert ok == 0
    # a gradient that is an input, two gradients in one buffer, a null pointer
    assert lib.wf2hip_attention_backward_f32(C.byref(d), p(x[0]), p(x[1]), p(x[2]), p(x[3]), p(x[4]), p(lse), p(x[0]),
                                             p(x[6]), p(x[7])) == W.lib.EOVERLAP
    assert lib.wf2hip_attention_backward_f32(C.byref(d), p(x[0]), p(x[1]), p(x[2]), p(x[3]), p(x[4]), p(lse), p(x[5]),
                                             p(x[5]), p(x[7])) == W.lib.EOVERLAP
    assert lib.wf2hip_attention_backward_f32(C.byref(d), p(x[0]), p(x[1]), p(x[2]), p(x[3]), p(x[4]), None, p(x[5]),
                                             p(x[6]), p(x[7])) == W.lib.EINVAL
    d.head_dim = 6
    assert lib.wf2hip_attention_backward_f32(C.byref(d), p(x[0]), p(x[1]), p(x[2]), p(x[3]), p(x[4]), p(lse), p(x[5]),
                                             p(x[6]), p(x[7])) == W.lib.EUNSUPPORTED
