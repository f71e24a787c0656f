"""Graph capture and replay of a node sequence (wf2hip_graph_*).

A replay must reproduce the eager result bit for bit on every launch, with the
program's own eager work and synchronisations between the replays, and must
follow new contents written into the captured input buffer."""
import importlib

import numpy as np
import pytest

from helpers import assert_bit_equal

pytestmark = pytest.mark.gpu

CFG = dict(batch=2, seq=40, d_model=64, n_head=2, head_dim=32, d_ff=96, eps=1e-5)


@pytest.mark.parametrize("mode", ["nodes", "fused"])
def test_block_forward_replay(gpu, mode):
    W = gpu
    F = W.functional
    gpt2 = importlib.import_module("cl-waffe2_amd.gpt2")
    params = gpt2.to_device(gpt2.make_block_params(3, CFG))
    x_host = gpt2.make_block_input(3, CFG)
    x = F.from_numpy(x_host)
    mask = gpt2.causal_mask(CFG["seq"])

    def run():
        return gpt2.block_forward(x, params, mode=mode, cfg=CFG, mask=mask)

    eager = run().numpy()            # also warms the pool with every temporary
    with W.lib.Graph() as g:
        out = run()
    for i in range(3):
        g.launch()
        assert_bit_equal(out.numpy(), eager, f"replay {i}")
        # eager work between replays, recycling pool blocks
        junk = F.exp(F.from_numpy(np.full((64, 64), float(i), np.float32)))
        assert junk.numpy()[0, 0] == np.float32(np.exp(np.float64(i)))
        W.lib.synchronize()
    # new contents in the same input buffer
    x2 = (x_host * np.float32(0.5) + np.float32(0.25)).astype(np.float32)
    F.move_(x, F.from_numpy(x2))
    g.launch()
    replayed = out.numpy()
    want = run().numpy()
    assert_bit_equal(replayed, want, "replay on new input")
    assert not np.array_equal(replayed, eager)
    g.destroy()


def test_scratch_using_kernels_replay(gpu):
    """Kernels that take scratch from the pool (column sums, split-K products) inside
    a recorded graph: every replay equals the eager result, also when the input changes."""
    W = gpu
    F = W.functional
    rng = np.random.default_rng(5)
    X = rng.standard_normal((4096, 320)).astype(np.float32)
    A = rng.standard_normal((96, 4096)).astype(np.float32)
    x, a = F.from_numpy(X), F.from_numpy(A)

    def run():
        return F.sum(x, axis=0), F.matmul(a, x)

    e_sum, e_mm = (t.numpy() for t in run())   # warms the pool with the scratch blocks
    with W.lib.Graph() as g:
        s, mm = run()
    for i in range(3):
        g.launch()
        assert_bit_equal(s.numpy(), e_sum, f"column sums, replay {i}")
        assert_bit_equal(mm.numpy(), e_mm, f"split-K product, replay {i}")
        junk = F.exp(F.from_numpy(np.full((4096, 320), 0.5, np.float32)))  # eager work between replays
        assert junk.numpy()[0, 0] == np.float32(np.exp(np.float64(0.5)))
    F.move_(x, F.from_numpy((X * np.float32(2.0)).astype(np.float32)))
    g.launch()
    w_sum, w_mm = (t.numpy() for t in run())
    assert_bit_equal(s.numpy(), w_sum, "column sums on new input")
    assert_bit_equal(mm.numpy(), w_mm, "split-K product on new input")
    g.destroy()


def test_capture_rules(gpu):
    W = gpu
    F = W.functional
    a = F.from_numpy(np.ones((33, 77), np.float32))
    with pytest.raises(W.HIPError) as e:
        with W.lib.Graph():
            F.exp(W.HIPTensor([12345, 7]))  # a size the pool has never seen: would need hipMalloc
    assert e.value.code == W.lib.ECAPTURE
    with pytest.raises(W.HIPError) as e:
        with W.lib.Graph():
            a.numpy()                        # a blocking host transfer
    assert e.value.code == W.lib.ECAPTURE
    lib = W.lib.get()
    import ctypes as C
    h = C.c_void_p()
    assert lib.wf2hip_graph_end(C.byref(h)) == W.lib.ECAPTURE   # nothing to end
    # the library still works afterwards
    assert F.add(a, a).numpy()[0, 0] == 2.0


def test_block_dropped_after_the_capture_stays_with_the_graph(gpu):
    """A result allocated during a capture and dropped after it (a host collector
    finalising it at any later time) must not go back to the pool while the graph
    lives: the next eager allocation of that size would receive the block every
    replay still writes into."""
    W = gpu
    F = W.functional
    n = 3 << 18  # its own size class, so that the pool holds exactly the blocks of this test
    x = F.from_numpy(np.full(n, 1.0, np.float32))
    warm = F.exp(x)          # the pool learns the size
    W.lib.synchronize()
    del warm
    with W.lib.Graph() as g:
        out = F.exp(x)       # served from the idle pool during the capture
    g.launch()
    W.lib.synchronize()
    idle_before = W.lib.get().wf2hip_pool_idle_bytes()
    del out                  # dropped after the capture
    assert W.lib.get().wf2hip_pool_idle_bytes() == idle_before, "the block went back to the idle pool"
    fresh = W.HIPTensor([n], initial_element=None)
    F.move_(fresh, F.from_numpy(np.full(n, 7.0, np.float32)))
    for _ in range(3):
        g.launch()
    W.lib.synchronize()
    assert np.all(fresh.numpy() == 7.0), "a replay wrote into a tensor allocated after the capture"
    parked = W.lib.get().wf2hip_pool_idle_bytes()
    g.destroy()
    assert W.lib.get().wf2hip_pool_idle_bytes() >= parked + 4 * n  # the parked block is back


def test_graph_released_during_a_recording(gpu):
    """A graph handle rebound while the next graph is being recorded (`with Graph() as g:` over an older g)
    releases the older graph inside the recording: its destruction waits for the end of the recording, and
    the new graph records and replays as usual."""
    W = gpu
    F = W.functional
    x = F.from_numpy(np.arange(4096, dtype=np.float32))

    def run():
        return F.exp(F.mul(x, 1.0 / 4096))

    eager = run().numpy()
    with W.lib.Graph() as g:
        first = run()
    g.launch()
    assert_bit_equal(first.numpy(), eager, "first graph")
    run()                          # the first graph keeps its blocks: the pool needs a set for the second
    with W.lib.Graph() as g:       # the first graph loses its last reference here, inside the recording
        second = run()
    for i in range(2):
        g.launch()
        assert_bit_equal(second.numpy(), eager, f"second graph, replay {i}")


@pytest.mark.parametrize("rows", [128, 256, 512])
def test_layer_replay_equals_eager_bit_for_bit(gpu, rows):
    """A Linear layer on a few hundred rows runs as slices of K folded in a fixed order, the slice count chosen
    from the shape (so its bits depend on the number of rows fed through it).  Captured after a warm-up, every
    replay must equal the eager result bit for bit: the route never depends on what the pool happens to hold."""
    W = gpu
    F = W.functional
    rng = np.random.default_rng(rows)
    x = F.from_numpy(rng.standard_normal((rows, 768)).astype(np.float32))
    w = F.from_numpy((0.02 * rng.standard_normal((768, 2304))).astype(np.float32))
    b = F.from_numpy(rng.standard_normal(2304).astype(np.float32))
    eager = F.linear(x, w, b, activation="gelu").numpy()
    with W.lib.Graph() as g:
        out = F.linear(x, w, b, activation="gelu")
    for i in range(2):
        g.launch()
        assert_bit_equal(out.numpy(), eager, f"rows {rows}, replay {i}")
    g.destroy()
    ref = x.numpy().astype(np.float64) @ w.numpy().astype(np.float64) + b.numpy()
    ref = 0.5 * ref * (1 + np.tanh(np.sqrt(2 / np.pi) * (ref + 0.044715 * ref ** 3)))
    assert np.abs(eager - ref).max() <= 2e-5 * max(1.0, np.abs(ref).max())


def test_capture_without_scratch_fails_loudly(gpu):
    """A product that splits K needs a scratch block.  Captured without a warm-up (the pool has never seen the
    block) it must fail with WF2HIP_ECAPTURE rather than quietly take another route with other rounding."""
    W = gpu
    F = W.functional
    rng = np.random.default_rng(11)
    # shapes of their own, so that no earlier test has left a matching scratch block in the pool
    x = F.from_numpy(rng.standard_normal((200, 1056)).astype(np.float32))
    w = F.from_numpy(rng.standard_normal((1056, 1000)).astype(np.float32))
    out = W.HIPTensor([200, 1000], initial_element=None)
    W.lib.check(W.lib.get().wf2hip_pool_trim())
    with pytest.raises(W.HIPError) as e:
        with W.lib.Graph():
            F.matmul(x, w, out=out)
    assert e.value.code == W.lib.ECAPTURE
    eager = F.matmul(x, w, out=out).numpy().copy()  # warm-up
    with W.lib.Graph() as g:
        F.matmul(x, w, out=out)
    g.launch()
    assert_bit_equal(out.numpy(), eager, "replay after the warm-up")
    g.destroy()
