"""The allocation-free row-sum entry point against the allocating one it mirrors.

wf2hip_reduce_add_rows_f32_noalloc keeps its partial sums in a static device
array that every call on the GPU shares, so the calls below come in pairs on
one stream, the second with a smaller input: what the first call left in the
array must not leak into the second.  Same kernels, same order of partial
sums: the bar is bit equality with wf2hip_reduce_add_rows_f32 (and <= 1e-5
relative to the sum of magnitudes against float64, the bar of every
reduction).
"""
import ctypes as C

import numpy as np
import pytest

from helpers import assert_bit_equal

pytestmark = pytest.mark.gpu


def dptr(t, offset=0):
    return C.c_void_p(t.ptr + 4 * offset)


def _both(W, x, ldx, rows, cols, start):
    lib = W.lib.get()
    dx = W.HIPTensor.from_numpy(x)
    got = W.HIPTensor.from_numpy(start.copy())
    want = W.HIPTensor.from_numpy(start.copy())
    W.lib.check(lib.wf2hip_reduce_add_rows_f32_noalloc(rows, cols, dptr(dx), ldx, dptr(got), 1))
    W.lib.check(lib.wf2hip_reduce_add_rows_f32(rows, cols, dptr(dx), ldx, dptr(want), 1))
    return got.numpy(), want.numpy()


# (rows, cols) pairs: the first of each pair splits its rows over many workgroups (fewer
# than 2048 rows: partial sums go through the scratch array), the second is smaller
@pytest.mark.parametrize("first, second", [
    ((64, 1 << 18), (3, 5000)),
    ((1, 1 << 22), (1, 70000)),
    ((500, 40000), (7, 33000)),
    ((4096, 4096), (17, 1000)),  # no split at all, then a short split one
])
def test_noalloc_matches_allocating_entry_twice_in_a_row(gpu, first, second):
    W = gpu
    rng = np.random.default_rng(7)
    for rows, cols in (first, second):
        print("case", rows, cols, flush=True)
        x = rng.standard_normal((rows, cols)).astype(np.float32)
        start = rng.standard_normal(rows).astype(np.float32)
        got, want = _both(W, x, cols, rows, cols, start)
        assert_bit_equal(got, want, f"rows {rows} cols {cols}")
        ref = start.astype(np.float64) + x.astype(np.float64).sum(axis=1)
        mag = np.abs(start).astype(np.float64) + np.abs(x).astype(np.float64).sum(axis=1)
        assert np.all(np.abs(got - ref) <= 1e-5 * mag)


def test_noalloc_padded_rows_and_single_column(gpu):
    W = gpu
    rng = np.random.default_rng(8)
    x = rng.standard_normal((37, 30000)).astype(np.float32)
    start = np.zeros(37, np.float32)
    got, want = _both(W, x, 30000, 37, 29999, start)  # ldx > cols: ragged, unaligned rows
    assert_bit_equal(got, want, "padded rows")
    got, want = _both(W, x, 30000, 37, 1, start)  # one column: a strided add
    assert_bit_equal(got, want, "single column")
    assert_bit_equal(got, x[:, 0], "single column value")


def test_noalloc_refuses_sizes_beyond_its_maximum(gpu):
    W = gpu
    lib = W.lib.get()
    d = W.HIPTensor([4])
    rc = lib.wf2hip_reduce_add_rows_f32_noalloc(1 << 20, 1 << 13, dptr(d), 1 << 13, dptr(d), 1)
    assert rc == W.lib.EUNSUPPORTED
    assert b"maximum" in lib.wf2hip_last_error()
    assert lib.wf2hip_reduce_add_rows_f32_noalloc(0, 5, None, 5, None, 1) == 0


@pytest.mark.parametrize("rows, cols, ldx, inco", [
    (64, 1 << 18, 1 << 18, 1),    # rows split over workgroups
    (4096, 4096, 4096, 1),        # a wavefront or workgroup per row
    (37, 29999, 30000, 1),        # padded rows
    (37, 1, 30000, 1),            # one column: a strided add
    (40, 50000, 50016, 0),        # every row into one number, padded rows: two reduced axes
    (40, 50000, 50000, 0),        # the same, dense: one long run
    (70000, 1, 3, 0),             # a strided column into one number
])
def test_noalloc_requests_no_block(gpu, rows, cols, ldx, inco):
    """No block is requested from the allocator, whatever form the arguments normalise to; results agree with
    the allocating entry to the bar of every reduction (bit equality where both run the same kernels)."""
    W = gpu
    lib = W.lib.get()
    rng = np.random.default_rng(9)
    x = rng.standard_normal((rows, ldx)).astype(np.float32)
    nout = rows if inco else 1
    start = rng.standard_normal(nout).astype(np.float32)
    dx = W.HIPTensor.from_numpy(x)
    got = W.HIPTensor.from_numpy(start.copy())
    want = W.HIPTensor.from_numpy(start.copy())
    W.lib.check(lib.wf2hip_sync())
    before = lib.wf2hip_pool_requests()
    W.lib.check(lib.wf2hip_reduce_add_rows_f32_noalloc(rows, cols, dptr(dx), ldx, dptr(got), inco))
    assert lib.wf2hip_pool_requests() == before, "the allocation-free entry point asked the allocator for a block"
    W.lib.check(lib.wf2hip_reduce_add_rows_f32(rows, cols, dptr(dx), ldx, dptr(want), inco))
    got, want = got.numpy(), want.numpy()
    x64 = x[:, :cols].astype(np.float64)
    if inco:
        assert_bit_equal(got, want, f"rows {rows} cols {cols} ldx {ldx}")
        ref, mag = start + x64.sum(axis=1), np.abs(start) + np.abs(x64).sum(axis=1)
    else:
        ref, mag = start + x64.sum(), np.abs(start) + np.abs(x64).sum()
        assert np.all(np.abs(want - ref) <= 1e-5 * mag)
    assert np.all(np.abs(got - ref) <= 1e-5 * mag)
