"""The allocator's bookkeeping (cl-waffe2_amd/csrc/wf2_pool.h) built for the CPU: which block is idle, and which
captured graphs keep a block they were recorded with.  The device runtime performs the allocations themselves;
everything decided here is decided the same way on the GPU.

The role of this pool is the one `maybe-allocate!` / `adjust-allocation!` have in the reference
(source/vm/allocation.lisp:71-145): temporaries are allocated once and reused."""
import ctypes as C
import os
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))


@pytest.fixture(scope="module")
def P():
    so = os.path.join(HERE, "native", "libwf2_pool_cpu.so")
    deps = [os.path.join(HERE, "native", "pool_cpu.cpp"), os.path.join(HERE, "..", "cl-waffe2_amd", "csrc", "wf2_pool.h")]
    if not os.path.exists(so) or os.path.getmtime(so) < max(os.path.getmtime(f) for f in deps):
        subprocess.check_call(["make", "-C", os.path.join(HERE, "native"), "-B"], stdout=subprocess.DEVNULL)
    L = C.CDLL(so)
    vp, ul = C.c_void_p, C.c_ulong
    for name, res, args in [("pool_new", vp, [C.c_int]), ("pool_delete", None, [vp]), ("graph_new", vp, []),
                            ("pool_alloc", vp, [vp, ul, vp]), ("pool_free", C.c_int, [vp, vp, vp]),
                            ("graph_destroy", C.c_int, [vp, vp]), ("pool_idle_bytes", ul, [vp]),
                            ("pool_blocks_known", ul, [vp]), ("pool_owners_of", ul, [vp, vp]),
                            ("graph_held", ul, [vp]), ("pool_size_class", ul, [ul])]:
        getattr(L, name).restype = res
        getattr(L, name).argtypes = args
    return L


KEPT, RELEASED = 1, 2


def test_size_classes(P):
    assert P.pool_size_class(1) == 512
    assert P.pool_size_class(512) == 512
    assert P.pool_size_class(513) == 1024
    assert P.pool_size_class((1 << 20) - 1) == 1 << 20
    assert P.pool_size_class(1 << 20) == 2 << 20
    assert P.pool_size_class((2 << 20) + 1) == 4 << 20


def test_recycling_without_graphs(P):
    pool = P.pool_new(1)
    a = P.pool_alloc(pool, 1000, None)
    assert P.pool_free(pool, a, None) == KEPT
    assert P.pool_idle_bytes(pool) == 1024
    assert P.pool_alloc(pool, 600, None) == a  # same size class: recycled
    assert P.pool_idle_bytes(pool) == 0
    b = P.pool_alloc(pool, 600, None)
    assert b != a
    assert P.pool_free(pool, 12345, None) == 0  # unknown pointer
    P.pool_free(pool, a, None)
    P.pool_free(pool, b, None)
    P.pool_delete(pool)


def test_capture_never_allocates(P):
    pool, g = P.pool_new(1), P.graph_new()
    assert P.pool_alloc(pool, 4096, g) is None
    P.graph_destroy(pool, g)
    P.pool_delete(pool)


def test_block_of_a_capture_waits_for_its_graph(P):
    pool = P.pool_new(1)
    warm = P.pool_alloc(pool, 4096, None)
    P.pool_free(pool, warm, None)
    g = P.graph_new()
    t = P.pool_alloc(pool, 4096, g)  # recorded with g
    assert t == warm and P.pool_owners_of(pool, t) == 1
    assert P.pool_free(pool, t, g) == KEPT and P.graph_held(g) == 1
    assert P.pool_alloc(pool, 4096, g) == t  # later allocation of the same capture
    # capture over; the host drops the result afterwards
    assert P.pool_free(pool, t, None) == KEPT
    assert P.pool_idle_bytes(pool) == 0 and P.graph_held(g) == 1
    assert P.pool_alloc(pool, 4096, None) != t  # an eager allocation never gets it
    assert P.graph_destroy(pool, g) == 0
    assert P.pool_idle_bytes(pool) == 4096
    P.pool_delete(pool)


@pytest.mark.parametrize("first_destroyed", ["A", "B"])
def test_block_of_two_graphs_waits_for_both(P, first_destroyed):
    """A block recorded into graph A and still held by the host is freed while graph B is being captured:
    it belongs to both, whichever is destroyed first."""
    pool = P.pool_new(1)
    warm = P.pool_alloc(pool, 8192, None)
    P.pool_free(pool, warm, None)
    A = P.graph_new()
    x = P.pool_alloc(pool, 8192, A)  # A's kernels write x; the host keeps it
    assert x == warm
    B = P.graph_new()
    assert P.pool_free(pool, x, B) == KEPT  # freed during B's capture (B's kernels read it)
    assert P.pool_owners_of(pool, x) == 2
    first, second = (A, B) if first_destroyed == "A" else (B, A)
    assert P.graph_destroy(pool, first) == 0
    assert P.pool_idle_bytes(pool) == 0, "the block went back to the pool while a graph still replays into it"
    assert P.pool_owners_of(pool, x) == 1 and P.graph_held(second) == 1
    assert P.pool_alloc(pool, 8192, None) != x
    assert P.graph_destroy(pool, second) == 0
    assert P.pool_idle_bytes(pool) == 8192 and P.pool_owners_of(pool, x) == 0
    assert P.pool_alloc(pool, 8192, None) == x
    P.pool_delete(pool)


def test_block_held_by_the_host_outlives_its_graph(P):
    pool = P.pool_new(1)
    warm = P.pool_alloc(pool, 2048, None)
    P.pool_free(pool, warm, None)
    g = P.graph_new()
    out = P.pool_alloc(pool, 2048, g)
    P.graph_destroy(pool, g)  # the host still holds `out`
    assert P.pool_owners_of(pool, out) == 0 and P.pool_idle_bytes(pool) == 0
    assert P.pool_free(pool, out, None) == KEPT
    assert P.pool_idle_bytes(pool) == 2048
    P.pool_delete(pool)


def test_disabled_pool_releases(P):
    pool = P.pool_new(0)
    a = P.pool_alloc(pool, 512, None)
    assert P.pool_free(pool, a, None) == RELEASED
    assert P.pool_blocks_known(pool) == 0
    # a block freed during a capture is still parked with the graph, and released with it
    b = P.pool_alloc(pool, 512, None)
    g = P.graph_new()
    assert P.pool_free(pool, b, g) == KEPT
    assert P.pool_alloc(pool, 512, g) == b
    assert P.pool_free(pool, b, g) == KEPT
    assert P.graph_destroy(pool, g) == 1
    assert P.pool_blocks_known(pool) == 0
    P.pool_delete(pool)
