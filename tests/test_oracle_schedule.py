"""Pins the oracle's restatement of cl-waffe2's loop scheduler
(solve-loop-order, do-compiled-loop.lisp:76-164; call-with-view.lisp:112-229):

* the schedules of the benchmark configurations, derived by hand from the
  reference source (flatten only when every tensor's remaining views are all T
  or all broadcast; otherwise batch loops and one call per innermost row);
* the invariant that the emitted 1-D calls touch every visible element exactly
  once;
* a brute-force N-D index walk on random tiny views, bit for bit.
"""
import itertools

import numpy as np
import pytest

from helpers import assert_bit_equal, host_tensor, oracle_views


def sched(O, *tensors, cap=1 << 17):
    return O.schedule(oracle_views(O, list(tensors)), cap=cap)


def test_config1_flattens(W, O):
    a, b = host_tensor(W, (1024, 1024)), host_tensor(W, (1024, 1024))
    cnt, calls = sched(O, a, b)
    assert cnt == 1 and calls[0] == (1 << 20, (0, 0), (1, 1))


def test_config2_row_broadcast_is_one_call_per_row(W, O):
    x = host_tensor(W, (4096, 8192))
    y = host_tensor(W, (1, 8192)).view((":broadcast", 4096), True)
    cnt, calls = sched(O, x, y)
    assert cnt == 4096
    assert calls[0] == (8192, (0, 0), (1, 1)) and calls[5] == (8192, (5 * 8192, 0), (1, 1))


def test_config2_strided_slice_copy_and_scalar_mul(W, O):
    src = host_tensor(W, (4096, 8192)).view(True, (0, 8192, 2))
    dst = host_tensor(W, (4096, 4096))
    cnt, calls = sched(O, dst, src)
    assert cnt == 4096 and calls[3] == (4096, (3 * 4096, 3 * 8192), (1, 2))
    s = host_tensor(W, (1, 1)).view((":broadcast", 4096), (":broadcast", 4096))
    cnt, calls = sched(O, dst, s)
    assert cnt == 1 and calls[0] == (1 << 24, (0, 0), (1, 0))


def test_config2_offset_views(W, O):
    A = host_tensor(W, (4096, 8192))
    x = host_tensor(W, (2048, 8192))
    y = A.view((0, 2048), True)
    cnt, calls = sched(O, x, y)
    assert cnt == 2048 and calls[7] == (8192, (7 * 8192, 7 * 8192), (1, 1))
    cnt, calls = sched(O, x, A.view((1024, 3072), True))
    assert cnt == 2048 and calls[0] == (8192, (0, 1024 * 8192), (1, 1))


def test_config4_reductions(W, O):
    a = host_tensor(W, (8192, 4096))
    out = host_tensor(W, (8192, 1)).view(True, (":broadcast", 4096))
    cnt, calls = sched(O, out, a)
    assert cnt == 8192 and calls[9] == (4096, (9, 9 * 4096), (0, 1))  # incx = 0: sequential accumulate
    full = host_tensor(W, (1, 1)).view((":broadcast", 8192), (":broadcast", 4096))
    cnt, calls = sched(O, full, a)
    assert cnt == 1 and calls[0] == (1 << 25, (0, 0), (0, 1))


def test_unary_flat(W, O):
    x, o = host_tensor(W, (1 << 13, 1 << 13)), host_tensor(W, (1 << 13, 1 << 13))
    cnt, calls = sched(O, x, o)
    assert cnt == 1 and calls[0] == (1 << 26, (0, 0), (1, 1))


def _random_sub(rng, n):
    k = rng.integers(0, 6)
    if k == 0 or n < 3:
        return True
    if k == 1:
        a = int(rng.integers(0, n - 1))
        return (a, int(rng.integers(a + 1, n + 1)))
    if k == 2:
        a = int(rng.integers(0, n - 2))
        return (a, int(rng.integers(a + 2, n + 1)), int(rng.integers(2, 4)))
    if k == 3:
        a = int(rng.integers(0, n - 2))
        return (a, int(rng.integers(a + 2, n + 1)), -int(rng.integers(1, 3)))
    if k == 4:
        return int(rng.integers(0, n))
    return True


def _random_pair(W, rng):
    rank = int(rng.integers(1, 5))
    storage = [int(rng.integers(1, 7)) for _ in range(rank)]
    x = host_tensor(W, storage).view(*[_random_sub(rng, n) for n in storage])
    vis = x.shape
    ystorage, ysubs = [], []
    for n in vis:
        if n > 1 and rng.random() < 0.35:
            ystorage.append(1)
            ysubs.append((":broadcast", n))
        else:
            pad = int(rng.integers(0, 3))
            ystorage.append(n + pad)
            ysubs.append((pad, n + pad) if pad else True)
    y = host_tensor(W, ystorage).view(*ysubs)
    if rng.random() < 0.3:  # make x the broadcast (accumulating) side instead
        x, y = y, x
    return x, y


@pytest.mark.parametrize("seed", range(8))
def test_calls_cover_every_element_once(W, O, seed):
    rng = np.random.default_rng(seed)
    for _ in range(60):
        x, y = _random_pair(W, rng)
        shape, sx, ox = x.geometry()
        _, sy, oy = y.geometry()
        cnt, calls = sched(O, x, y)
        assert cnt == len(calls)
        for t, (strides, off) in enumerate(((sx, ox), (sy, oy))):
            want = {}
            for idx in itertools.product(*[range(n) for n in shape]):
                o = off + sum(i * s for i, s in zip(idx, strides))
                want[o] = want.get(o, 0) + 1
            got = {}
            for n, offs, incs in calls:
                for i in range(n):
                    o = offs[t] + i * incs[t]
                    got[o] = got.get(o, 0) + 1
            assert got == want, (x, y, t)
        assert sum(c[0] for c in calls) == int(np.prod(shape))


@pytest.mark.parametrize("seed", range(8))
def test_node_nd_equals_naive_index_walk(W, O, seed):
    """x <- x op y executed through the schedule equals a row-major walk over
    the visible index space (sequential semantics, including accumulation into
    broadcast destinations)."""
    rng = np.random.default_rng(100 + seed)
    ops = {"add": np.add, "sub": np.subtract, "mul": np.multiply, "div": np.divide}
    for _ in range(40):
        x, y = _random_pair(W, rng)
        shape, sx, ox = x.geometry()
        _, sy, oy = y.geometry()
        xs = rng.uniform(0.5, 1.5, x.vec.nbytes // 4).astype(np.float32)
        ys = rng.uniform(0.9, 1.1, y.vec.nbytes // 4).astype(np.float32)
        name = list(ops)[int(rng.integers(0, 4))]
        got = xs.copy()
        O.node_nd(name, oracle_views(O, [x, y]), got, ys.copy())
        want = xs.copy()
        for idx in itertools.product(*[range(n) for n in shape]):
            i = ox + sum(a * s for a, s in zip(idx, sx))
            j = oy + sum(a * s for a, s in zip(idx, sy))
            want[i] = ops[name](want[i], ys[j])
        assert_bit_equal(got, want, f"{name} {x} {y}")
        # MoveTensorNode: last write wins on broadcast destinations
        got = xs.copy()
        O.node_nd("move", oracle_views(O, [x, y]), got, ys.copy())
        want = xs.copy()
        for idx in itertools.product(*[range(n) for n in shape]):
            want[ox + sum(a * s for a, s in zip(idx, sx))] = ys[oy + sum(a * s for a, s in zip(idx, sy))]
        assert_bit_equal(got, want, f"move {x} {y}")
