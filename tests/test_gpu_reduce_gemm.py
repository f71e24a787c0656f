"""GPU parity of reductions, softmax, LayerNorm and gemm.

Bar: <= 1e-5 relative error for reductions and gemm
(relative to the sum of magnitudes, because a sum of N(0,1) values is itself
~0); bit-exact against the oracle in the sequential reduce mode; the
reference's own integer test vectors exactly.
"""
import ctypes as C

import numpy as np
import pytest

from helpers import assert_bit_equal, oracle_views, ulp_distance

pytestmark = pytest.mark.gpu

REL = 1e-5


def dptr(t, offset=0):
    return C.c_void_p(t.ptr + 4 * offset)


def test_sum_tester_vectors(gpu):
    """sum-tester / mean-tester of the reference
    (base-impl/t/reduction.lisp:9-48): ones(100,100,100) -> 1e6 for axis t,
    100 for axis 0 / 1 / -1, 10000 for axes (0 1); mean -> 1.0."""
    F = gpu.functional
    ones = F.make_tensor((100, 100, 100), initial_element=1.0)
    assert F.sum(ones).numpy().ravel().tolist() == [1000000.0]
    for axis in (0, 1, -1):
        out = F.sum(ones, axis=axis)
        assert out.size == 10000 and np.all(out.numpy() == 100.0)
    out = F.sum(ones, axis=(0, 1))
    assert out.shape == [1, 1, 100] and np.all(out.numpy() == 10000.0)
    assert np.all(F.mean(ones, axis=1).numpy() == 1.0)
    assert F.mean(ones).numpy().ravel().tolist() == [1.0]
    kd = F.sum(ones, axis=1, keepdims=True)
    assert kd.shape == [100, 100, 100] and np.all(kd.numpy() == 100.0)


def test_sums_over_leading_axes(gpu):
    """!sum over the leading axes with the last axis kept (bias gradients): the column
    form, whole vectors and ragged column counts, one and several reduced axes, a
    sliced source; float64 truth, 1e-5 relative to the sum of magnitudes."""
    W = gpu
    F = W.functional
    rng = np.random.default_rng(101)
    for shape, axis in [((3000, 768), 0), ((17, 1000), 0), ((64, 50, 260), (0, 1)), ((4100, 67), 0),
                        ((9, 33, 1030), (0, 1)), ((20000, 64), 0)]:
        X = rng.standard_normal(shape).astype(np.float32)
        got = F.sum(F.from_numpy(X), axis=axis).numpy()
        want = X.astype(np.float64).sum(axis=axis, keepdims=True)
        scale = np.abs(X).astype(np.float64).sum(axis=axis, keepdims=True)
        assert got.shape == want.shape
        assert np.max(np.abs(got - want) / scale) < 1e-5, (shape, axis)
    X = rng.standard_normal((5000, 512)).astype(np.float32)
    v = F.from_numpy(X).view((100, 4100), (3, 259))
    got = F.sum(v, axis=0).numpy()
    want = X[100:4100, 3:259].astype(np.float64).sum(axis=0, keepdims=True)
    assert np.max(np.abs(got - want)) < 1e-3
    # accumulation adds to what the destination holds
    acc = F.from_numpy(np.full((1, 512), 2.5, np.float32))
    F.add_(acc.view((":broadcast", 5000), True), F.from_numpy(X))
    np.testing.assert_allclose(acc.numpy(), 2.5 + X.astype(np.float64).sum(axis=0, keepdims=True), rtol=0, atol=2e-3)


def test_many_short_rows(gpu):
    """Row sums of many rows of at most 512 elements (four rows per wavefront), with
    row lengths that are not multiples of four through a view: float64 truth, 1e-5
    relative to the sum of magnitudes."""
    W = gpu
    F = W.functional
    rng = np.random.default_rng(97)
    for rows, pitch, cols in [(10000, 256, 256), (9000, 512, 512), (8200, 100, 100), (12000, 256, 250),
                              (9001, 384, 321), (8192, 4, 4)]:
        X = rng.standard_normal((rows, pitch)).astype(np.float32)
        v = F.from_numpy(X).view(True, (0, cols))
        got = F.sum(v, axis=1).numpy()
        want = X[:, :cols].astype(np.float64).sum(axis=1, keepdims=True)
        scale = np.abs(X[:, :cols]).astype(np.float64).sum(axis=1, keepdims=True)
        assert got.shape == want.shape
        assert np.max(np.abs(got - want) / scale) < 1e-5, (rows, pitch, cols)
        mean = F.mean(v, axis=1).numpy()
        assert np.max(np.abs(mean - want / cols) / (scale / cols)) < 1e-5


def test_config4_row_and_full_sum(gpu, O):
    """benchmark configuration 4: row sum and full sum of (8192, 4096) N(0,1), seed 4.
    Tree mode against float64 truth; a slice of it in sequential mode against
    the oracle's strictly ordered fp32 accumulation, bit for bit."""
    W = gpu
    F = W.functional
    rng = np.random.Generator(np.random.PCG64(4))
    A = rng.standard_normal((8192, 4096)).astype(np.float32)
    dA = F.from_numpy(A)
    A64 = A.astype(np.float64)
    mag_rows = np.abs(A64).sum(axis=1)
    got = F.sum(dA, axis=1).numpy().ravel()
    assert np.all(np.abs(got - A64.sum(axis=1)) <= REL * mag_rows)
    got = F.sum(dA).numpy().ravel()[0]
    assert abs(got - A64.sum()) <= REL * np.abs(A64).sum()
    # the GPU tree result must also be at least as close to the truth as the
    # reference's own sequential fp32 order is
    seq = np.zeros(1, np.float32)
    O.binary_1d("add", A.size, seq, 0, A.ravel(), 1)
    assert abs(got - A64.sum()) <= abs(float(seq[0]) - A64.sum()) + 1e-3

    lib = W.lib.get()
    W.lib.check(lib.wf2hip_set_reduce_mode(1))
    try:
        small = dA.view((0, 64), True)
        got = F.sum(small, axis=1).numpy().ravel()
        want = np.zeros(64, np.float32)
        for r in range(64):
            O.binary_1d("add", 4096, want, 0, A[r], 1, offx=r)
        assert_bit_equal(got, want, "sequential row sums")
        got = F.sum(small).numpy().ravel()
        want = np.zeros(1, np.float32)
        O.binary_1d("add", 64 * 4096, want, 0, np.ascontiguousarray(A[:64]).ravel(), 1)
        assert_bit_equal(got, want, "sequential full sum")
    finally:
        W.lib.check(lib.wf2hip_set_reduce_mode(0))


@pytest.mark.parametrize("shape,axis", [((7, 13), 1), ((7, 13), 0), ((5, 6, 7), (0, 2)), ((5, 6, 7), 1),
                                        ((3000,), True), ((1, 70000), 1), ((3, 1 << 18), 1),
                                        ((2, 3, 4, 5), (1, 3)), ((300, 300), True), ((64, 1000), 0),
                                        ((513, 2049), 1), ((4, 5000, 3), 1)])
def test_reduce_shapes(gpu, shape, axis):
    """Row, column, mixed and split-row reductions against float64."""
    F = gpu.functional
    rng = np.random.default_rng(42)
    x = rng.standard_normal(shape).astype(np.float32)
    npaxis = None if axis is True else axis
    want = x.astype(np.float64).sum(axis=npaxis, keepdims=True)
    mag = np.abs(x.astype(np.float64)).sum(axis=npaxis, keepdims=True)
    got = F.sum(F.from_numpy(x), axis=axis).numpy()
    assert got.shape == want.shape
    assert np.all(np.abs(got - want) <= REL * mag)
    gotm = F.mean(F.from_numpy(x), axis=axis).numpy()
    cnt = x.size / want.size
    assert np.all(np.abs(gotm - want / cnt) <= REL * mag / cnt + 1e-7)


@pytest.mark.parametrize("shape, axis", [
    ((8192, 512), 1), ((64, 40000), 1), ((3, 70001), -1), ((1, 1 << 21), True), ((700, 300), True),
    ((3000, 768), 0), ((17, 1000), 0), ((64, 50, 260), (0, 1)), ((12, 33, 64), 1), ((5, 7, 9, 11), (1, 3)),
    ((100, 1), 1), ((1, 100), 1), ((6, 1, 8), 1), ((262144, 16), 1),
])
def test_one_node_sum_equals_the_composition(gpu, shape, axis):
    """!sum / !mean as ONE node (HIP-Sum-Node, wf2hip_sum_nd) against the reference's
    composition (zero fill by MulNode, AddNode into the broadcast view, DivNode) on the
    same input: bit-identical in both reduce modes, also when `out` holds stale NaNs
    (the one-node form never reads it), with and without keepdims."""
    W = gpu
    F = W.functional
    rng = np.random.default_rng(11)
    x = rng.standard_normal(shape).astype(np.float32)
    dx = F.from_numpy(x)
    assert F.ENABLE_SYMBOLIC_PATH
    for mode in (0, 1):
        if mode == 1 and x.size > (1 << 21):
            continue
        W.lib.check(W.lib.get().wf2hip_set_reduce_mode(mode))
        try:
            want = F.sum_composed(dx, axis=axis).numpy()
            assert_bit_equal(F.sum(dx, axis=axis).numpy(), want, f"sum {shape} {axis} mode {mode}")
            stale = F.from_numpy(np.full(want.shape, np.nan, np.float32))
            got = F.sum(dx, axis=axis, out=stale, keepdims=True)
            assert got.shape == list(shape)
            assert_bit_equal(stale.numpy(), want, "sum into a NaN-filled out")
            n = x.size // want.size
            wantm = F.sum_composed(dx, axis=axis, div_by=float(n)).numpy()
            assert_bit_equal(F.mean(dx, axis=axis).numpy(), wantm, f"mean {shape} {axis} mode {mode}")
        finally:
            W.lib.check(W.lib.get().wf2hip_set_reduce_mode(0))
    ref = x.astype(np.float64).sum(axis=None if axis is True else axis, keepdims=True)
    mag = np.abs(x).astype(np.float64).sum(axis=None if axis is True else axis, keepdims=True)
    assert np.all(np.abs(F.sum(dx, axis=axis).numpy() - ref) <= REL * mag)


def test_one_node_sum_on_views_and_switch(gpu):
    """Sliced sources, an `out` that is itself a view, and the switch back to the
    composition (ENABLE_SYMBOLIC_PATH, the mirror of *enable-symbolic-path*)."""
    W = gpu
    F = W.functional
    rng = np.random.default_rng(12)
    X = rng.standard_normal((300, 520)).astype(np.float32)
    v = F.from_numpy(X).view((10, 290), (3, 515))
    assert_bit_equal(F.sum(v, axis=1).numpy(), F.sum_composed(v, axis=1).numpy(), "sliced rows")
    assert_bit_equal(F.sum(v, axis=0).numpy(), F.sum_composed(v, axis=0).numpy(), "sliced columns")
    big = F.from_numpy(np.full((280, 4), 7.0, np.float32))
    out = big.view(True, (2, 3))
    F.sum(v, axis=1, out=out)
    want = big.numpy().copy()
    assert np.all(want[:, [0, 1, 3]] == 7.0)  # the neighbours of the viewed column are untouched
    assert_bit_equal(want[:, 2:3], F.sum_composed(v, axis=1).numpy(), "out as a view")
    F.ENABLE_SYMBOLIC_PATH = False
    try:
        assert_bit_equal(F.sum(v, axis=1).numpy(), F.sum_composed(v, axis=1).numpy(), "composition")
    finally:
        F.ENABLE_SYMBOLIC_PATH = True
    # integer and :double tensors keep the composition (HIP-Sum-Node is :float only)
    xi = F.from_numpy(np.arange(24, dtype=np.int32).reshape(4, 6), dtype="int32")
    assert F.sum(xi, axis=1).numpy().ravel().tolist() == [15, 51, 87, 123]


def test_accumulate_adds_to_existing_value(gpu):
    """AddNode into a stride-0 destination is x += sum(y), not x = sum(y)."""
    W = gpu
    x = W.HIPTensor.from_numpy(np.array([[10.0], [20.0]], np.float32))
    y = W.HIPTensor.from_numpy(np.arange(12, dtype=np.float32).reshape(2, 6))
    W.forward("AddNode", x.view(True, (":broadcast", 6)), y)
    assert x.numpy().ravel().tolist() == [25.0, 71.0]
    out = np.zeros(3, np.float32) + 5
    d = W.HIPTensor.from_numpy(out)
    W.lib.check(W.lib.get().wf2hip_reduce_add_rows_f32(3, 4, dptr(W.HIPTensor.from_numpy(np.ones((3, 4), np.float32))),
                                                      4, dptr(d), 1))
    assert d.numpy().tolist() == [9.0, 9.0, 9.0]


def test_max_min(gpu, O):
    W = gpu
    rng = np.random.default_rng(3)
    for n, inc in [(1, 1), (5, 1), (8, 1), (1000, 1), (1000, 3), (100000, 1), (3000000, 1)]:
        x = rng.standard_normal(n * inc).astype(np.float32)
        dx = W.HIPTensor.from_numpy(x)
        out = W.HIPTensor([1])
        W.lib.check(W.lib.get().wf2hip_smax(n, dptr(dx), inc, dptr(out)))
        assert out.numpy()[0] == O.maxmin_1d("max", n, x, inc) == x[::inc][:n].max()
        W.lib.check(W.lib.get().wf2hip_smin(n, dptr(dx), inc, dptr(out)))
        assert out.numpy()[0] == O.maxmin_1d("min", n, x, inc) == x[::inc][:n].min()


def _softmax64(x):
    x = x.astype(np.float64)
    e = np.exp(x - x.max(axis=-1, keepdims=True))
    return e / e.sum(axis=-1, keepdims=True)


def _assert_softmax(got, want64, what=""):
    """The fused kernel's bound: exp(x - max) carries the binary32 rounding of
    x - max (|x - max| 2^-24 relative: 4e-6 at the underflow edge) plus a few ulp
    of the exponential, the row sum and the final product; the bar for this
    configuration is 1e-5 relative.  Results below the normal range are flushed
    to zero (atol)."""
    np.testing.assert_allclose(got, want64, rtol=4e-6, atol=1.2e-38, err_msg=what)


def test_config4_softmax(gpu):
    """benchmark configuration 4: max-subtracted row softmax of (32768, 1024) N(0, 3^2)
    logits, seed 4 -- fused kernel against the float64 closed form; invariants
    of the reference's tests (rows sum to 1, nn/t/activation.lisp:9-12) and
    shift invariance."""
    W = gpu
    F = W.functional
    rng = np.random.Generator(np.random.PCG64(4))
    rng.standard_normal((8192, 4096))  # config 4 draws the sum tensor first
    X = (rng.standard_normal((32768, 1024)) * 3.0).astype(np.float32)
    got = F.softmax_fused(F.from_numpy(X)).numpy()
    want = _softmax64(X)
    _assert_softmax(got, want, "config 4")
    assert np.abs(got / want - 1.0)[want > 1e-30].mean() < 4e-7  # typical error: a few ulp
    assert np.abs(got.astype(np.float64).sum(axis=1) - 1.0).max() < 1e-5
    shifted = F.softmax_fused(F.from_numpy(X[:256] + np.float32(8.0))).numpy()
    np.testing.assert_allclose(shifted, _softmax64(X[:256] + np.float32(8.0)), rtol=1e-5, atol=1e-12)


@pytest.mark.parametrize("cols", [1, 3, 64, 100, 255, 256, 1000, 1024, 2050, 4096, 4097, 5000, 8192, 8193, 20000,
                                  32768, 40000, 50257, 53249, 65536, 70000, 200001])
def test_softmax_widths(gpu, cols):
    """Every row form: 1 ... 4096 columns in a wavefront's registers, 4097 ... 65536 in those of a workgroup of
    1024 threads (8, 16, 32, 52 or 64 elements per thread; a few rows beyond 16384 columns in pieces of 16384),
    longer rows in pieces."""
    F = gpu.functional
    rng = np.random.default_rng(cols)
    X = (rng.standard_normal((37 if cols < 30000 else 5, cols)) * 4).astype(np.float32)
    got = F.softmax_fused(F.from_numpy(X)).numpy()
    _assert_softmax(got, _softmax64(X), f"{cols} columns")


@pytest.mark.parametrize("rows,cols", [(300, 4100), (260, 8195), (258, 16384), (257, 20001), (260, 32770), (260, 50257),
                                       (257, 53248), (257, 53249), (256, 65536), (258, 65535)])
def test_softmax_a_workgroup_per_row(gpu, rows, cols):
    """At least a row per compute unit and 4097 ... 65536 columns: a workgroup of 1024 threads per row holding
    2, 4, 8, 13 or 16 vectors of four columns per thread, rows that start off a 16-byte boundary (odd lengths),
    lengths that are no multiple of four, and the largest row of every form."""
    F = gpu.functional
    rng = np.random.default_rng(rows * 31 + cols)
    X = (rng.standard_normal((rows, cols)) * 3).astype(np.float32)
    X[0, cols - 1] = 30.0          # the maximum in the last column
    X[1, : cols // 2] = -np.inf    # half a row that contributes nothing
    got = F.softmax_fused(F.from_numpy(X)).numpy()
    _assert_softmax(got, _softmax64(X), f"({rows}, {cols})")
    assert np.abs(got.astype(np.float64).sum(axis=1) - 1.0).max() < 1e-5


@pytest.mark.parametrize("rows,cols", [(1, 16385), (1, 1 << 22), (3, 16384 * 5 + 7), (300, 32768), (300, 70001), (2, 1234567)])
def test_softmax_rows_in_pieces(gpu, rows, cols):
    """Rows handled as pieces of 16384 columns whose maxima and sums are folded afterwards: pieces that hold the
    row's maximum first, last and in the middle, a piece of -inf only, a ragged last piece, in place, and an
    unaligned row pitch; rows sum to 1."""
    F = gpu.functional
    rng = np.random.default_rng(rows + cols)
    X = (rng.standard_normal((rows, cols)) * 3).astype(np.float32)
    X[0, cols - 1] = 30.0                       # the maximum in the last piece
    if rows > 1:
        X[1, 0] = 40.0                          # ... in the first
        X[1, 16384:min(cols, 32768)] = -np.inf  # a piece that contributes nothing
    d = F.from_numpy(X)
    got = F.softmax_fused(d).numpy()
    _assert_softmax(got, _softmax64(X), f"({rows}, {cols})")
    assert np.abs(got.astype(np.float64).sum(axis=1) - 1.0).max() < 1e-5
    F.softmax_fused(d, out=d)  # in place: always the two launches, whose pieces are shorter
    np.testing.assert_allclose(d.numpy(), got, rtol=8e-6, atol=1.2e-38)  # each within 4e-6 of the truth
    _assert_softmax(d.numpy(), _softmax64(X), f"({rows}, {cols}) in place")


def test_softmax_long_rows_in_one_launch(gpu, monkeypatch):
    """A few rows whose pieces of 65536 columns all fit on the device at once go through one launch in which
    every workgroup waits for the others' statistics: (1, 2^24) is one workgroup on every compute unit.  Twice in
    a row and then a smaller one (the counters of the meeting are left at zero by each launch); the same with
    no polls allowed, where every workgroup takes the path of one that gave up waiting and works out the row's
    statistics by itself."""
    F = gpu.functional
    rng = np.random.default_rng(24)
    big = (rng.standard_normal((1, 1 << 24)) * 3).astype(np.float32)
    big[0, 12345678] = 25.0
    want_big = _softmax64(big)
    d, o = F.from_numpy(big), gpu.HIPTensor([1, 1 << 24])
    for _ in range(2):
        F.softmax_fused(d, out=o)
        _assert_softmax(o.numpy(), want_big, "(1, 2^24)")
    small = (rng.standard_normal((3, 65536 * 3 + 8)) * 3).astype(np.float32)
    small[1, :65536] = -np.inf
    want_small = _softmax64(small)
    got = F.softmax_fused(F.from_numpy(small)).numpy()
    _assert_softmax(got, want_small, "(3, 196616)")
    assert np.abs(got.astype(np.float64).sum(axis=1) - 1.0).max() < 1e-5
    monkeypatch.setenv("WF2HIP_MEET_SPINS", "0")
    alone = F.softmax_fused(F.from_numpy(small)).numpy()
    _assert_softmax(alone, want_small, "(3, 196616), nobody waits")
    monkeypatch.delenv("WF2HIP_MEET_SPINS")
    again = F.softmax_fused(F.from_numpy(small)).numpy()
    np.testing.assert_array_equal(again, got)


def test_softmax_reference_composition(gpu, O):
    """!softmax exactly as the reference composes it (mean-subtract, axis 1):
    each node against the oracle running the same node on the CPU."""
    W = gpu
    F = W.functional
    rng = np.random.default_rng(9)
    X = rng.standard_normal((64, 96)).astype(np.float32)
    got = F.softmax(F.from_numpy(X)).numpy()
    # oracle: same decomposition, sequential CPU semantics
    s = np.zeros(64, np.float32)
    for r in range(64):
        O.binary_1d("add", 96, s, 0, X[r], 1, offx=r)
    mean = s / np.float32(96.0)
    x1 = X - mean[:, None]
    e = np.zeros_like(x1)
    O.unary_1d("exp", x1.size, x1.ravel(), 1, e.reshape(-1), 1)
    z = np.zeros(64, np.float32)
    for r in range(64):
        O.binary_1d("add", 96, z, 0, e[r], 1, offx=r)
    want = e / z[:, None]
    np.testing.assert_allclose(got, want, rtol=2e-6, atol=1e-9)
    np.testing.assert_allclose(got, _softmax64(X), rtol=1e-5)
    assert np.abs(got.sum(axis=1) - 1).max() < 1e-5


def test_causal_softmax(gpu):
    W = gpu
    rng = np.random.default_rng(6)
    for batch, seq in [(3, 64), (2, 100), (2, 1024), (1, 7)]:
        X = rng.standard_normal((batch, seq, seq)).astype(np.float32) * 5
        scale = np.float32(0.125)
        dx = W.HIPTensor.from_numpy(X)
        out = W.HIPTensor(X.shape)
        W.lib.check(W.lib.get().wf2hip_causal_softmax_f32(batch, seq, dptr(dx), dptr(out), float(scale)))
        s = (X * scale).astype(np.float64)
        mask = np.tril(np.ones((seq, seq), bool))
        s = np.where(mask, s, -np.inf)
        want = _softmax64(s)
        got = out.numpy()
        assert np.all(got[:, ~mask] == 0.0)
        _assert_softmax(got, want, f"causal {batch}x{seq}")


def test_layernorm(gpu):
    """Fused LayerNorm against float64, and the node-for-node recipe of
    LayerNorm-Revisit (examples/gpt-2/utils.lisp:114-127) against it."""
    W = gpu
    F = W.functional
    rng = np.random.default_rng(7)
    # 2052 ... 8192 (multiples of 4): a workgroup per row holding it in registers; 4101: three passes;
    # beyond 8192: the row in pieces of 16384 columns over several workgroups
    for rows, cols in [(64, 768), (10, 100), (5, 1), (33, 2048), (7, 255), (9, 3072), (3, 4101), (2, 20000),
                       (1001, 1024), (513, 1000), (300, 1536), (5, 2052), (300, 4096), (7, 5120), (40, 6148),
                       (129, 8192), (3, 8196), (700, 8200), (5, 16384), (3, 16388), (2, 40001), (1, (1 << 20) + 4),
                       (40, 32768)]:
        X = (rng.standard_normal((rows, cols)) * 2 + 0.5).astype(np.float32)
        g = rng.standard_normal(cols).astype(np.float32)
        b = rng.standard_normal(cols).astype(np.float32)
        X64 = X.astype(np.float64)
        mu = X64.mean(axis=1, keepdims=True)
        var = ((X64 - mu) ** 2).mean(axis=1, keepdims=True)
        want = (X64 - mu) / np.sqrt(var + 1e-5) * g + b
        got = F.layer_norm_fused(F.from_numpy(X), F.from_numpy(g), F.from_numpy(b)).numpy()
        np.testing.assert_allclose(got, want, rtol=2e-6, atol=2e-6)
        got = F.layer_norm(F.from_numpy(X), F.from_numpy(g), F.from_numpy(b)).numpy()
        np.testing.assert_allclose(got, want, rtol=1e-4, atol=1e-4)


def test_layernorm_long_rows_in_one_launch(gpu, monkeypatch):
    """A few rows whose pieces of 65536 columns all fit on the device at once: one launch in which every workgroup
    waits for the others' statistics.  (1, 2^24) fills the device; twice in a row, then a smaller one (the counters
    of the meeting are left at zero), then with no polls allowed: every workgroup works out the row's statistics by
    itself.  Against float64."""
    F = gpu.functional
    rng = np.random.default_rng(42)

    def check(X, g, b, what):
        X64 = X.astype(np.float64)
        mu = X64.mean(axis=1, keepdims=True)
        var = ((X64 - mu) ** 2).mean(axis=1, keepdims=True)
        want = (X64 - mu) / np.sqrt(var + 1e-5) * g + b
        got = F.layer_norm_fused(F.from_numpy(X), F.from_numpy(g), F.from_numpy(b)).numpy()
        np.testing.assert_allclose(got, want, rtol=2e-6, atol=2e-6, err_msg=what)
        return got

    n = 1 << 24
    X = (rng.standard_normal((1, n)) * 2 + 0.5).astype(np.float32)
    g = rng.standard_normal(n).astype(np.float32)
    b = rng.standard_normal(n).astype(np.float32)
    for _ in range(2):
        check(X, g, b, "(1, 2^24)")
    del X, g, b
    cols = 65536 * 3 + 8
    X = (rng.standard_normal((3, cols)) * 3 - 1.0).astype(np.float32)
    g = rng.standard_normal(cols).astype(np.float32)
    b = rng.standard_normal(cols).astype(np.float32)
    first = check(X, g, b, "(3, 196616)")
    monkeypatch.setenv("WF2HIP_MEET_SPINS", "0")
    check(X, g, b, "(3, 196616), nobody waits")
    monkeypatch.delenv("WF2HIP_MEET_SPINS")
    again = check(X, g, b, "(3, 196616) again")
    np.testing.assert_array_equal(again, first)


# ---------------------------------------------------------------------------
# gemm
# ---------------------------------------------------------------------------

def test_matmul_reference_vectors(gpu):
    """matmul-tester, -mnk, -mnk1, matmul-both-transposed
    (base-impl/t/arithmetic.lisp:116-149): integer-valued, exact under any
    correct gemm."""
    F = gpu.functional
    a33 = F.from_numpy(np.arange(9, dtype=np.float32).reshape(3, 3))
    a34 = F.from_numpy(np.arange(12, dtype=np.float32).reshape(3, 4))
    assert F.matmul(a33, a33).numpy().ravel().tolist() == [15, 18, 21, 42, 54, 66, 69, 90, 111]
    assert F.matmul(a34, F.t(a34)).numpy().ravel().tolist() == [14, 38, 62, 38, 126, 214, 62, 214, 366]
    assert F.matmul(F.t(a34), a34).numpy().ravel().tolist() == [80, 92, 104, 116, 92, 107, 122, 137, 104, 122,
                                                               140, 158, 116, 137, 158, 179]
    assert F.matmul(F.t(a33), F.t(a33)).numpy().ravel().tolist() == [15, 42, 69, 18, 54, 90, 21, 66, 111]


def _gemm_check(got, A64, B64):
    want = A64 @ B64
    bound = REL * (np.abs(A64) @ np.abs(B64)) + 1e-30
    assert np.all(np.abs(got - want) <= bound), float(np.max(np.abs(got - want) / bound))


@pytest.mark.parametrize("m,n,k", [(1, 1, 1), (3, 5, 7), (128, 128, 16), (129, 127, 33), (256, 384, 64),
                                   (100, 260, 1000), (64, 64, 4), (512, 768, 768), (1000, 10, 3), (2, 300, 130)])
@pytest.mark.parametrize("ta,tb", [(False, False), (True, False), (False, True), (True, True)])
def test_matmul_random(gpu, m, n, k, ta, tb):
    F = gpu.functional
    rng = np.random.default_rng(m * 7 + n * 3 + k)
    A = rng.standard_normal((m, k)).astype(np.float32)
    B = rng.standard_normal((k, n)).astype(np.float32)
    dA = F.t(F.from_numpy(np.ascontiguousarray(A.T))) if ta else F.from_numpy(A)
    dB = F.t(F.from_numpy(np.ascontiguousarray(B.T))) if tb else F.from_numpy(B)
    got = F.matmul(dA, dB).numpy()
    _gemm_check(got, A.astype(np.float64), B.astype(np.float64))


@pytest.mark.parametrize("ta,tb", [(False, False), (True, False), (False, True), (True, True)])
def test_matmul_few_tiles_long_k(gpu, ta, tb):
    """Products with few output tiles and a long K (weight gradients) run split over K
    and are folded afterwards: every layout, leading dimensions and beta through the
    column-major entry point as well."""
    W = gpu
    F = W.functional
    rng = np.random.default_rng(303 + ta + 2 * tb)
    # the last four: tiny outputs over a very long K (the weight gradients of layers with few outputs),
    # which run as up to 1024 slices folded by a wavefront per output element
    for m, n, k in [(768, 640, 8192), (200, 300, 4096), (130, 1000, 2048), (10, 256, 65536), (256, 10, 65536),
                    (4, 9, 100352), (3, 3, 1 << 20), (127, 127, 100000), (33, 65, 5003), (200, 100, 2049),
                    (5, 7, 300001)]:   # the last four: K that no equal slices divide, a shorter last slice
        A = rng.standard_normal((m, k)).astype(np.float32)
        B = rng.standard_normal((k, n)).astype(np.float32)
        dA = F.t(F.from_numpy(np.ascontiguousarray(A.T))) if ta else F.from_numpy(A)
        dB = F.t(F.from_numpy(np.ascontiguousarray(B.T))) if tb else F.from_numpy(B)
        _gemm_check(F.matmul(dA, dB).numpy(), A.astype(np.float64), B.astype(np.float64))
    # one batch level of such products, K on and off equal slices
    for batch, m, n, k in [(12, 3, 5, 100000), (5, 130, 40, 4096), (3, 64, 64, 6001)]:
        A = rng.standard_normal((batch, m, k)).astype(np.float32)
        B = rng.standard_normal((batch, k, n)).astype(np.float32)
        dA = F.t(F.from_numpy(np.ascontiguousarray(A.transpose(0, 2, 1)))) if ta else F.from_numpy(A)
        dB = F.t(F.from_numpy(np.ascontiguousarray(B.transpose(0, 2, 1)))) if tb else F.from_numpy(B)
        got = F.matmul(dA, dB).numpy()
        for b in range(batch):
            _gemm_check(got[b], A[b].astype(np.float64), B[b].astype(np.float64))
    # column-major contract with beta and padded leading dimensions
    lib = W.lib.get()
    m, n, k = 96, 200, 4096
    ca, cb = ("T" if ta else "N"), ("T" if tb else "N")
    lda = (m if ca == "N" else k) + 4
    ldb = (k if cb == "N" else n) + 8
    ldc = m + 4
    A = rng.standard_normal(lda * (k if ca == "N" else m)).astype(np.float32)
    B = rng.standard_normal(ldb * (n if cb == "N" else k)).astype(np.float32)
    Cm = rng.standard_normal(ldc * n).astype(np.float32)
    A2 = A.reshape(-1, lda).T.astype(np.float64)  # column-major storage: lda rows
    B2 = B.reshape(-1, ldb).T.astype(np.float64)
    opA = A2[:m, :k] if ca == "N" else A2[:k, :m].T
    opB = B2[:k, :n] if cb == "N" else B2[:n, :k].T
    C2 = Cm.reshape(-1, ldc).T.astype(np.float64)
    want = C2.copy()
    want[:m, :n] = 0.5 * opA @ opB - 2.0 * C2[:m, :n]
    dA, dB, dC = W.HIPTensor.from_numpy(A), W.HIPTensor.from_numpy(B), W.HIPTensor.from_numpy(Cm)
    W.lib.check(lib.wf2hip_sgemm(ca.encode(), cb.encode(), m, n, k, 0.5, dptr(dA), lda, dptr(dB), ldb, -2.0,
                                 dptr(dC), ldc))
    got = dC.numpy().reshape(-1, ldc).T
    scale = 0.5 * np.abs(opA) @ np.abs(opB) + 2.0 * np.abs(C2[:m, :n])
    assert np.max(np.abs(got[:m, :n] - want[:m, :n]) / scale) < 1e-5
    np.testing.assert_array_equal(got[m:, :], C2[m:, :].astype(np.float32))  # padding rows untouched


def test_sgemm_column_major_contract(gpu, O):
    """wf2hip_sgemm keeps Fortran sgemm_ semantics (column-major, alpha/beta,
    leading dimensions larger than the matrix), checked against the oracle's
    netlib restatement."""
    W = gpu
    rng = np.random.default_rng(77)
    lib = W.lib.get()
    for ta, tb in [("N", "N"), ("T", "N"), ("N", "T"), ("T", "T")]:
        m, n, k = 37, 29, 53
        lda = (m if ta == "N" else k) + 3
        ldb = (k if tb == "N" else n) + 5
        ldc = m + 2
        A = rng.standard_normal(lda * (k if ta == "N" else m)).astype(np.float32)
        B = rng.standard_normal(ldb * (n if tb == "N" else k)).astype(np.float32)
        Cm = rng.standard_normal(ldc * n).astype(np.float32)
        want = Cm.copy()
        O.sgemm(ta, tb, m, n, k, 0.75, A, lda, B, ldb, -1.5, want, ldc)
        dA, dB, dC = W.HIPTensor.from_numpy(A), W.HIPTensor.from_numpy(B), W.HIPTensor.from_numpy(Cm)
        W.lib.check(lib.wf2hip_sgemm(ta.encode(), tb.encode(), m, n, k, 0.75, dptr(dA), lda, dptr(dB), ldb,
                                     -1.5, dptr(dC), ldc))
        got = dC.numpy()
        np.testing.assert_allclose(got, want, rtol=1e-4, atol=1e-4)
        # padding rows of C (ldc > m) are never written
        pad = np.arange(got.size) % ldc >= m
        assert_bit_equal(got[pad], Cm[pad], "ldc padding")
    # beta == 0 must not read C (NaN in C stays out of the result)
    nanC = W.HIPTensor.from_numpy(np.full(16, np.nan, np.float32))
    eye = W.HIPTensor.from_numpy(np.eye(4, dtype=np.float32).ravel())
    W.lib.check(lib.wf2hip_sgemm(b"N", b"N", 4, 4, 4, 1.0, dptr(eye), 4, dptr(eye), 4, 0.0, dptr(nanC), 4))
    assert nanC.numpy().tolist() == np.eye(4).ravel().tolist()
    assert lib.wf2hip_sgemm(b"X", b"N", 4, 4, 4, 1.0, dptr(eye), 4, dptr(eye), 4, 0.0, dptr(nanC), 4) == -1
    assert lib.wf2hip_sgemm(b"N", b"N", 4, 4, 4, 1.0, dptr(eye), 2, dptr(eye), 4, 0.0, dptr(nanC), 4) == -1


def test_matmul_batched_and_broadcast(gpu):
    """Batch axes, a rank-2 weight against a rank-3 activation (the !flexible
    broadcast of nn/regression.lisp:14-18), permuted head layouts."""
    F = gpu.functional
    rng = np.random.default_rng(31)
    X = rng.standard_normal((4, 50, 24)).astype(np.float32)
    Wt = rng.standard_normal((24, 36)).astype(np.float32)
    got = F.matmul(F.from_numpy(X), F.from_numpy(Wt)).numpy()
    for b in range(4):
        _gemm_check(got[b], X[b].astype(np.float64), Wt.astype(np.float64))
    Q = rng.standard_normal((2, 3, 40, 16)).astype(np.float32)
    K = rng.standard_normal((2, 3, 40, 16)).astype(np.float32)
    got = F.matmul(F.from_numpy(Q), F.t(F.from_numpy(K))).numpy()
    assert got.shape == (2, 3, 40, 40)
    for b in range(2):
        for h in range(3):
            _gemm_check(got[b, h], Q[b, h].astype(np.float64), K[b, h].T.astype(np.float64))
    # heads read straight out of a fused (B, T, 3, H, hd) projection: batch
    # strides that do not merge -> host loop over the outer batch axis
    qkv = rng.standard_normal((2, 40, 3, 3, 16)).astype(np.float32)
    d = F.from_numpy(qkv)
    q = d.view(True, True, 0, True, True)
    q = F.reshape(F.copy(q.permute(0, 2, 3, 1, 4)), 2, 3, 40, 16)
    got = F.matmul(q, F.t(q)).numpy()
    for b in range(2):
        for h in range(3):
            M = qkv[b, :, 0, h, :].astype(np.float64)
            _gemm_check(got[b, h], M, M.T)


def test_matmul_fused_epilogue_against_the_node_sequence(gpu):
    """act(a @ w + bias) + residual in the gemm epilogue against MatMulNode,
    AddNode, fused GELU kernel, AddNode run one after the other: bit-identical
    for bias and residual; the epilogue's GELU is the binary32 form (v_exp_f32,
    v_rcp_f32) and stays within 4e-6 relative of the binary64 one (plus half an
    ulp of the residual sum)."""
    F = gpu.functional
    rng = np.random.default_rng(51)
    for shape_a, n in [((3, 70, 48), 100), ((130, 64), 256), ((2, 2, 33, 20), 7)]:
        a = rng.standard_normal(shape_a).astype(np.float32)
        w = (rng.standard_normal((shape_a[-1], n)) * 0.2).astype(np.float32)
        bias = rng.standard_normal(n).astype(np.float32)
        res = rng.standard_normal(shape_a[:-1] + (n,)).astype(np.float32)
        da, dw, db, dr = (F.from_numpy(v) for v in (a, w, bias, res))
        plain = F.add_(F.matmul(da, dw), db)
        assert_bit_equal(F.matmul(da, dw, bias=db).numpy(), plain.numpy(), "bias")
        act = F.gelu_fused(plain)
        got = F.matmul(da, dw, bias=db, activation="gelu").numpy()
        np.testing.assert_allclose(got, act.numpy(), rtol=4e-6, atol=1e-37, err_msg="bias+gelu")
        assert np.abs(got / np.where(act.numpy() == 0, 1, act.numpy()) - 1).mean() < 3e-7
        want = F.add(plain, dr)
        assert_bit_equal(F.matmul(da, dw, bias=db, residual=dr).numpy(), want.numpy(), "bias+residual")
        want = F.add(act, dr)
        got = F.matmul(da, dw, bias=db, activation="gelu", residual=dr).numpy()
        np.testing.assert_allclose(got, want.numpy(), rtol=0,
                                   atol=4e-6 * np.abs(act.numpy()).max() + 1.2e-7 * np.abs(want.numpy()).max(),
                                   err_msg="bias+gelu+residual")


def test_matmul_causal_modes(gpu):
    """causal=1: the lower triangle of q k^T equals the full product's (entries
    above the diagonal are unspecified); causal=2: a lower-triangular left
    operand gives the full product."""
    F = gpu.functional
    rng = np.random.default_rng(52)
    for t, hd in [(300, 16), (128, 64), (129, 8), (1024, 64)]:
        q = rng.standard_normal((2, 3, t, hd)).astype(np.float32)
        k = rng.standard_normal((2, 3, t, hd)).astype(np.float32)
        v = rng.standard_normal((2, 3, t, hd)).astype(np.float32)
        dq, dk, dv = F.from_numpy(q), F.from_numpy(k), F.from_numpy(v)
        full = F.matmul(dq, F.t(dk)).numpy()
        tri = F.matmul(dq, F.t(dk), causal=1).numpy()
        low = np.tril(np.ones((t, t), bool))
        assert_bit_equal(tri[..., low], full[..., low], f"lower triangle t={t}")
        p = np.tril(rng.standard_normal((2, 3, t, t))).astype(np.float32)
        dp = F.from_numpy(p)
        assert_bit_equal(F.matmul(dp, dv, causal=2).numpy(), F.matmul(dp, dv).numpy(), f"triangular left t={t}")
    with pytest.raises(gpu.HIPError):
        F.matmul(F.from_numpy(q[0, 0]), F.from_numpy(np.ones((hd, 5), np.float32)), causal=1)

@pytest.mark.parametrize("tile", ["w", "n", "x", "t"])
@pytest.mark.parametrize("tb", [False, True])
def test_matmul_streaming_kernel_matches_register_staged_kernel(gpu, monkeypatch, tile, tb):
    """K a multiple of 32 (from 256 on, or always with WF2HIP_GEMM_STREAM=1) and
    aligned operands takes the global->LDS streaming kernel; it contracts k in the same order as the register-staged kernel, so
    the two are bit-identical.  Ragged M / N (clamped loads), both tile widths,
    both right-operand layouts, bias + GELU + residual, and sgemm_ with beta."""
    import ctypes as C
    W = gpu
    F = W.functional
    rng = np.random.default_rng(77 + tb)
    monkeypatch.setenv("WF2HIP_GEMM_TILE", tile)
    for m, n, k in [(128, 128, 32), (200, 132, 96), (1, 4, 64), (515, 260, 416), (64, 1024, 128)]:
        A = rng.standard_normal((m, k)).astype(np.float32)
        B = rng.standard_normal((k, n)).astype(np.float32)
        bias = rng.standard_normal(n).astype(np.float32)
        res = rng.standard_normal((m, n)).astype(np.float32)
        dA = F.from_numpy(A)
        dB = F.t(F.from_numpy(np.ascontiguousarray(B.T))) if tb else F.from_numpy(B)
        db, dr = F.from_numpy(bias), F.from_numpy(res)
        outs = {}
        for mode in ("stream", "staged"):
            monkeypatch.setenv("WF2HIP_GEMM_STREAM", "0" if mode == "staged" else "1")
            outs[mode] = (F.matmul(dA, dB).numpy(),
                          F.matmul(dA, dB, bias=db, activation="gelu", residual=dr).numpy())
        monkeypatch.delenv("WF2HIP_GEMM_STREAM", raising=False)
        _gemm_check(outs["stream"][0], A.astype(np.float64), B.astype(np.float64))
        assert_bit_equal(outs["stream"][0], outs["staged"][0], f"plain {m}x{n}x{k}")
        assert_bit_equal(outs["stream"][1], outs["staged"][1], f"fused {m}x{n}x{k}")
    # Fortran contract with beta and a padded ldc (odd pitch: scalar stores)
    m, n, k = 100, 36, 64
    for ldc in (m + 3, m + 4):
        A = rng.standard_normal((k, m)).astype(np.float32)      # column-major m x k, lda = m
        B = rng.standard_normal((n, k)).astype(np.float32)      # column-major k x n, ldb = k
        Cm = rng.standard_normal((n, ldc)).astype(np.float32)
        dA, dB = W.HIPTensor.from_numpy(A), W.HIPTensor.from_numpy(B)
        got = {}
        for mode in ("stream", "staged"):
            monkeypatch.setenv("WF2HIP_GEMM_STREAM", "0" if mode == "staged" else "1")
            dC = W.HIPTensor.from_numpy(Cm)
            W.lib.check(W.lib.get().wf2hip_sgemm(b"N", b"N", m, n, k, 0.5, C.c_void_p(dA.ptr), m,
                                                 C.c_void_p(dB.ptr), k, -2.0, C.c_void_p(dC.ptr), ldc))
            got[mode] = dC.numpy()
        monkeypatch.delenv("WF2HIP_GEMM_STREAM", raising=False)
        want = Cm.astype(np.float64)                               # the padding is left alone
        want[:, :m] = -2.0 * want[:, :m] + 0.5 * (B.astype(np.float64) @ A.astype(np.float64))
        np.testing.assert_allclose(got["stream"], want, rtol=0, atol=1e-4)
        assert_bit_equal(got["stream"], got["staged"], f"sgemm beta ldc={ldc}")


def test_matmul_gelu_epilogue_edge_values(gpu):
    """The binary32 GELU of the gemm epilogue on inputs that reach its edges: a
    1 x 1 product carries each value through; float64 closed form."""
    F = gpu.functional
    xs = np.array([0.0, -0.0, 1.0, -1.0, 3.0, -3.0, 5.5, -5.5, 9.0, -9.0, 12.0, -12.0, 40.0, -40.0, 1e-8, -1e-8,
                   1e-30, 3e4, -3e4, 1e30, -1e30, np.inf, -np.inf, np.nan], np.float32)
    a = np.zeros((xs.size, 32), np.float32)
    a[:, 0] = xs
    w = np.zeros((32, 4), np.float32)
    w[0, :] = 1.0
    got = F.matmul(F.from_numpy(a), F.from_numpy(w), activation="gelu").numpy()[:, 0]
    x64 = xs.astype(np.float64)
    with np.errstate(all="ignore"):
        # 0.5 x (1 + tanh u) = x / (1 + exp(-2 u)); the left form cancels for u << 0
        truth = x64 / (1.0 + np.exp(-2.0 * np.sqrt(2.0 / np.pi) * (x64 + 0.044715 * x64 ** 3)))
    truth[xs == -np.inf] = -0.0
    finite = np.isfinite(truth)
    np.testing.assert_allclose(got[finite], truth[finite], rtol=4e-6, atol=1e-37)
    assert got[xs == np.inf][0] == np.inf and np.isnan(got[-1])
    assert got[xs == -np.inf][0] == 0.0 and got[list(xs).index(np.float32(-1e30))] == 0.0


@pytest.mark.parametrize("rows", [1, 2, 7, 16, 17, 32, 33, 64])
@pytest.mark.parametrize("cols,k", [(256, 64), (300, 100), (1000, 768), (5003, 260), (4096, 4100), (50257, 768), (8200, 4100)])
def test_matmul_few_rows(gpu, rows, cols, k):
    """At most 64 rows against a wide operand (a few tokens through a layer) take the kernel that reads the
    wide operand once: both storages of it ((k, cols), and (cols, k) through !t), ragged column groups, K on
    and off the slices and the 16-step, and the fused epilogue (bias, GELU, residual) on the same path."""
    F = gpu.functional
    rng = np.random.default_rng(rows * 1000003 + cols * 7 + k)
    X = rng.standard_normal((rows, k)).astype(np.float32)
    Wkn = rng.standard_normal((k, cols)).astype(np.float32)
    dX = F.from_numpy(X)
    _gemm_check(F.matmul(dX, F.from_numpy(Wkn)).numpy(), X.astype(np.float64), Wkn.astype(np.float64))
    dWt = F.from_numpy(np.ascontiguousarray(Wkn.T))
    _gemm_check(F.matmul(dX, F.t(dWt)).numpy(), X.astype(np.float64), Wkn.astype(np.float64))
    if cols <= 5003:
        bias = rng.standard_normal(cols).astype(np.float32)
        res = rng.standard_normal((rows, cols)).astype(np.float32)
        z = X.astype(np.float64) @ Wkn.astype(np.float64) + bias
        bound = REL * (np.abs(X.astype(np.float64)) @ np.abs(Wkn.astype(np.float64)) + np.abs(bias)) + 1e-30
        got = F.linear(dX, F.from_numpy(Wkn), F.from_numpy(bias), residual=F.from_numpy(res)).numpy()
        assert np.all(np.abs(got - (z + res)) <= bound + REL * np.abs(res))
        got = F.linear(dX, F.from_numpy(Wkn), F.from_numpy(bias), activation="gelu").numpy()
        gelu = 0.5 * z * (1.0 + np.tanh(np.sqrt(2.0 / np.pi) * (z + 0.044715 * z ** 3)))
        assert np.all(np.abs(got - gelu) <= 2.0 * bound + 4e-6 * np.abs(gelu) + 1e-6)


@pytest.mark.parametrize("rows", [1, 9, 16, 25, 32])
@pytest.mark.parametrize("cols,k", [(32768, 64), (40001, 100), (50257, 768), (33000, 1028)])
def test_matmul_few_rows_against_a_table_of_many_rows(gpu, rows, cols, k):
    """At most 32 rows against a table of 32768 rows and more stored (cols, k) -- GPT-2's token projection,
    `(!matmul x (!t wte))`: a wavefront per 32 columns with the whole of K.  Ragged last group, K on and off the
    steps of 64, and the fused epilogue on the same path; float64 with the bound of the other gemm tests."""
    F = gpu.functional
    rng = np.random.default_rng(rows * 31 + cols + k)
    X = rng.standard_normal((rows, k)).astype(np.float32)
    Wt = rng.standard_normal((cols, k)).astype(np.float32)
    dX, dW = F.from_numpy(X), F.from_numpy(Wt)
    X64, W64 = X.astype(np.float64), Wt.astype(np.float64).T
    _gemm_check(F.matmul(dX, F.t(dW)).numpy(), X64, W64)
    bias = rng.standard_normal(cols).astype(np.float32)
    res = rng.standard_normal((rows, cols)).astype(np.float32)
    z = X64 @ W64 + bias
    bound = REL * (np.abs(X64) @ np.abs(W64) + np.abs(bias)) + 1e-30
    got = F.matmul(dX, F.t(dW), bias=F.from_numpy(bias), residual=F.from_numpy(res)).numpy()
    assert np.all(np.abs(got - (z + res)) <= bound + REL * np.abs(res))
    got = F.matmul(dX, F.t(dW), bias=F.from_numpy(bias), activation="gelu").numpy()
    gelu = 0.5 * z * (1.0 + np.tanh(np.sqrt(2.0 / np.pi) * (z + 0.044715 * z ** 3)))
    assert np.all(np.abs(got - gelu) <= 2.0 * bound + 4e-6 * np.abs(gelu) + 1e-6)


@pytest.mark.parametrize("rows", [33, 48, 64])
@pytest.mark.parametrize("cols,k", [(1024, 256), (4100, 768), (2051, 512), (2048, 4096), (50257, 768)])
def test_matmul_33_to_64_rows_against_a_table(gpu, rows, cols, k):
    """33 ... 64 rows against a weight stored (cols, k) (`(!matmul x (!t w))`, the token projection of the GPT-2
    example, examples/gpt-2/model.lisp:137-196) run with the operands exchanged through the streaming kernel,
    whose tiles are turned over on the way out: ragged last tiles, column counts that rule out 16-byte stores,
    few tiles over a long K (slices of K first), and the fused epilogue -- bias per column of the row-major
    product, GELU, residual -- on that path; all against float64 at the bar of every product."""
    F = gpu.functional
    rng = np.random.default_rng(rows * 7919 + cols + k)
    X = rng.standard_normal((rows, k)).astype(np.float32)
    Wt = (rng.standard_normal((cols, k)) / np.sqrt(k)).astype(np.float32)
    X64, W64 = X.astype(np.float64), Wt.astype(np.float64).T
    dX, dW = F.from_numpy(X), F.from_numpy(Wt)
    _gemm_check(F.matmul(dX, F.t(dW)).numpy(), X64, W64)
    if cols > 5000:
        return
    bias = rng.standard_normal(cols).astype(np.float32)
    res = rng.standard_normal((rows, cols)).astype(np.float32)
    z = X64 @ W64 + bias
    bound = REL * (np.abs(X64) @ np.abs(W64) + np.abs(bias)) + 1e-30
    got = F.matmul(dX, F.t(dW), bias=F.from_numpy(bias), residual=F.from_numpy(res)).numpy()
    assert np.all(np.abs(got - (z + res)) <= bound + REL * np.abs(res))
    got = F.matmul(dX, F.t(dW), bias=F.from_numpy(bias), activation="gelu").numpy()
    gelu = 0.5 * z * (1.0 + np.tanh(np.sqrt(2.0 / np.pi) * (z + 0.044715 * z ** 3)))
    assert np.all(np.abs(got - gelu) <= 2.0 * bound + 4e-6 * np.abs(gelu) + 1e-6)
    # an output that is a window of a wider tensor (rows of padding stay untouched) and starts off a 16-byte boundary
    wide = F.from_numpy(np.full((rows, cols + 5), 7.0, np.float32))
    F.matmul(dX, F.t(dW), out=wide.view(True, (1, cols + 1)))
    got = wide.numpy()
    _gemm_check(got[:, 1:cols + 1], X64, W64)
    assert np.all(got[:, 0] == 7.0) and np.all(got[:, cols + 1:] == 7.0)


def test_sgemm_few_rows_column_major_contract(gpu):
    """The same kernel through wf2hip_sgemm: column-major C (m x n, n <= 64) with padded leading dimensions,
    alpha and beta, both storages of A; rows of padding stay untouched."""
    W = gpu
    lib = W.lib.get()
    rng = np.random.default_rng(64)
    for ca in "NT":
        m, n, k = 1028, 5, 520
        lda = (m if ca == "N" else k) + 4
        ldb, ldc = k + 8, m + 3
        A = rng.standard_normal(lda * (k if ca == "N" else m)).astype(np.float32)
        B = rng.standard_normal(ldb * n).astype(np.float32)
        Cm = rng.standard_normal(ldc * n).astype(np.float32)
        A2 = A.reshape(-1, lda).T.astype(np.float64)
        B2 = B.reshape(-1, ldb).T.astype(np.float64)
        opA = A2[:m, :k] if ca == "N" else A2[:k, :m].T
        opB = B2[:k, :n]
        C2 = Cm.reshape(-1, ldc).T.astype(np.float64)
        dA, dB, dC = W.HIPTensor.from_numpy(A), W.HIPTensor.from_numpy(B), W.HIPTensor.from_numpy(Cm)
        W.lib.check(lib.wf2hip_sgemm(ca.encode(), b"N", m, n, k, 0.5, dptr(dA), lda, dptr(dB), ldb, -2.0, dptr(dC), ldc))
        got = dC.numpy().reshape(-1, ldc).T
        want = 0.5 * opA @ opB - 2.0 * C2[:m, :n]
        scale = 0.5 * np.abs(opA) @ np.abs(opB) + 2.0 * np.abs(C2[:m, :n])
        assert np.max(np.abs(got[:m, :n] - want) / scale) < 1e-5
        np.testing.assert_array_equal(got[m:, :], C2[m:, :].astype(np.float32))


@pytest.mark.parametrize("rows,k,cols", [(96, 768, 2304), (256, 768, 768), (256, 3072, 768), (130, 1024, 1000),
                                         (512, 800, 260), (300, 2080, 515)])
def test_linear_of_a_few_hundred_rows(gpu, rows, k, cols):
    """A layer applied to a few hundred rows: few output tiles over a K of several hundred, which runs as
    slices of K whose fold applies the bias, the GELU and the residual -- against float64, and bit for bit
    against the same product with its epilogue taken node for node (the fold adds what the nodes add)."""
    F = gpu.functional
    rng = np.random.default_rng(rows + k + cols)
    X = rng.standard_normal((rows, k)).astype(np.float32)
    Wm = (rng.standard_normal((k, cols)) * 0.05).astype(np.float32)
    bias = rng.standard_normal(cols).astype(np.float32)
    res = rng.standard_normal((rows, cols)).astype(np.float32)
    dX, dW, db, dr = F.from_numpy(X), F.from_numpy(Wm), F.from_numpy(bias), F.from_numpy(res)
    z = X.astype(np.float64) @ Wm.astype(np.float64) + bias
    bound = REL * (np.abs(X.astype(np.float64)) @ np.abs(Wm.astype(np.float64)) + np.abs(bias)) + 1e-30
    plain = F.matmul(dX, dW)
    _gemm_check(plain.numpy(), X.astype(np.float64), Wm.astype(np.float64))
    got = F.linear(dX, dW, db, residual=dr).numpy()
    assert np.all(np.abs(got - (z + res)) <= bound + REL * np.abs(res))
    assert_bit_equal(got, F.add_(F.add_(plain, db), dr).numpy(), "bias and residual in the fold against the nodes")
    got = F.linear(dX, dW, db, activation="gelu").numpy()
    gelu = 0.5 * z * (1.0 + np.tanh(np.sqrt(2.0 / np.pi) * (z + 0.044715 * z ** 3)))
    assert np.all(np.abs(got - gelu) <= 2.0 * bound + 4e-6 * np.abs(gelu) + 1e-6)


@pytest.mark.parametrize("seed", range(48))
def test_matmul_random_shapes_and_layouts(gpu, seed):
    """Random extents (1, a few, just past a tile, hundreds, thousands), transposes, an optional batch and an
    optional fused epilogue: whatever route the product takes (tiles, slices of K with the fold, the
    few-rows kernel, batches) is held to the same bound against float64."""
    F = gpu.functional
    rng = np.random.default_rng(9000 + seed)
    mn = [1, 2, 7, 16, 33, 64, 65, 128, 200, 256, 300, 1000, 2304]
    ks = [1, 4, 17, 64, 100, 256, 768, 1024, 2049, 3072, 5000]
    while True:
        m, n, k = int(rng.choice(mn)), int(rng.choice(mn)), int(rng.choice(ks))
        batch = int(rng.choice([0, 0, 1, 3]))
        if 2.0 * m * n * k * max(batch, 1) <= 3e9:
            break
    ta, tb = bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
    lead = (batch,) if batch else ()
    A = rng.standard_normal(lead + (m, k)).astype(np.float32)
    B = rng.standard_normal(lead + (k, n)).astype(np.float32)
    swap = lambda a: np.ascontiguousarray(np.swapaxes(a, -1, -2))  # noqa: E731
    dA = F.t(F.from_numpy(swap(A))) if ta else F.from_numpy(A)
    dB = F.t(F.from_numpy(swap(B))) if tb else F.from_numpy(B)
    A64, B64 = A.astype(np.float64), B.astype(np.float64)
    want = A64 @ B64
    bound = REL * (np.abs(A64) @ np.abs(B64)) + 1e-30
    got = F.matmul(dA, dB).numpy()
    assert got.shape == want.shape
    assert np.all(np.abs(got - want) <= bound), (m, n, k, batch, ta, tb, float(np.max(np.abs(got - want) / bound)))
    if not batch:
        bias = rng.standard_normal(n).astype(np.float32)
        res = rng.standard_normal((m, n)).astype(np.float32)
        got = F.matmul(dA, dB, bias=F.from_numpy(bias), residual=F.from_numpy(res)).numpy()
        assert np.all(np.abs(got - (want + bias + res)) <= bound + REL * (np.abs(bias) + np.abs(res))), (m, n, k, ta, tb)


@pytest.mark.parametrize("rows,cols,k", [(4, 9, 173056), (16, 100, 43264), (1, 1, 8192), (64, 64, 9000), (7, 73, 8200), (2, 190, 9000),
                                         (3, 3, 100001)])
def test_matmul_small_output_long_k_both_k_major(gpu, rows, cols, k):
    """x^T . y with x (k, rows) and y (k, cols): a small output over a long K with both operands stored K-major
    (the weight gradient of a convolution with few channels) -- workgroups over slices of K, outputs in
    registers, planes folded in a fixed order; also with alpha, beta and padded leading dimensions through
    wf2hip_sgemm."""
    W = gpu
    F = W.functional
    rng = np.random.default_rng(rows + cols + k)
    X = rng.standard_normal((k, rows)).astype(np.float32)
    Y = rng.standard_normal((k, cols)).astype(np.float32)
    got = F.matmul(F.t(F.from_numpy(X)), F.from_numpy(Y)).numpy()
    _gemm_check(got, X.T.astype(np.float64), Y.astype(np.float64))
    # column-major: C (cols x rows, ldc padded) <- 0.5 A B^T - 2 C with A (cols x k, lda) and B (rows x k, ldb)
    lib = W.lib.get()
    lda, ldb, ldc = cols + 3, rows + 2, cols + 1
    A = rng.standard_normal(lda * k).astype(np.float32)
    B = rng.standard_normal(ldb * k).astype(np.float32)
    Cm = rng.standard_normal(ldc * rows).astype(np.float32)
    A2 = A.reshape(k, lda).T.astype(np.float64)[:cols]       # cols x k
    B2 = B.reshape(k, ldb).T.astype(np.float64)[:rows]       # rows x k
    C2 = Cm.reshape(rows, ldc).T.astype(np.float64)
    dA, dB, dC = W.HIPTensor.from_numpy(A), W.HIPTensor.from_numpy(B), W.HIPTensor.from_numpy(Cm)
    W.lib.check(lib.wf2hip_sgemm(b"N", b"T", cols, rows, k, 0.5, dptr(dA), lda, dptr(dB), ldb, -2.0, dptr(dC), ldc))
    got = dC.numpy().reshape(rows, ldc).T
    want = 0.5 * A2 @ B2.T - 2.0 * C2[:cols]
    scale = 0.5 * np.abs(A2) @ np.abs(B2.T) + 2.0 * np.abs(C2[:cols])
    assert np.max(np.abs(got[:cols] - want) / scale) < 1e-5
    np.testing.assert_array_equal(got[cols:], C2[cols:].astype(np.float32))


@pytest.mark.parametrize("batch,m,n,k", [(65535, 8, 8, 8), (4096, 16, 16, 16), (1024, 3, 3, 1000), (300, 1, 1, 4096),
                                         (2000, 10, 10, 10), (100, 32, 32, 50), (64, 16, 16, 200), (256, 2, 1, 5000)])
@pytest.mark.parametrize("ta,tb", [(False, False), (True, False), (False, True), (True, True)])
def test_matmul_many_small_matrices(gpu, batch, m, n, k, ta, tb):
    """Batches of products with a few output elements each: an output element per thread, or per wavefront
    over a longer K; every transpose form, and a two-level batch with a broadcast right operand."""
    F = gpu.functional
    rng = np.random.default_rng(batch + m + n + k)
    A = rng.standard_normal((batch, m, k)).astype(np.float32)
    B = rng.standard_normal((batch, k, n)).astype(np.float32)
    swap = lambda a: np.ascontiguousarray(np.swapaxes(a, -1, -2))  # noqa: E731
    dA = F.t(F.from_numpy(swap(A))) if ta else F.from_numpy(A)
    dB = F.t(F.from_numpy(swap(B))) if tb else F.from_numpy(B)
    got = F.matmul(dA, dB).numpy()
    A64, B64 = A.astype(np.float64), B.astype(np.float64)
    want = A64 @ B64
    bound = REL * (np.abs(A64) @ np.abs(B64)) + 1e-30
    assert np.all(np.abs(got - want) <= bound)
    if batch % 4 == 0 and not ta:
        A4 = A.reshape(4, batch // 4, m, k)
        got = F.matmul(F.from_numpy(A4), dB.tensor if False else (F.t(F.from_numpy(swap(B[0]))) if tb else F.from_numpy(B[0]))).numpy()
        want = A4.astype(np.float64) @ B64[0]
        assert np.all(np.abs(got - want) <= REL * (np.abs(A4.astype(np.float64)) @ np.abs(B64[0])) + 1e-30)
