"""Shared helpers of the test-suite."""
import numpy as np


def bits(a):
    return np.ascontiguousarray(a, np.float32).view(np.uint32)


def assert_bit_equal(got, want, what=""):
    """Bitwise equality, except that any NaN matches any NaN (x86 and gfx950
    may differ in NaN payload/sign)."""
    got = np.ascontiguousarray(got, np.float32)
    want = np.ascontiguousarray(want, np.float32)
    assert got.shape == want.shape, (what, got.shape, want.shape)
    both_nan = np.isnan(got) & np.isnan(want)
    neq = (bits(got) != bits(want)) & ~both_nan
    if neq.any():
        i = np.flatnonzero(neq.ravel())[:5]
        raise AssertionError(f"{what}: {neq.sum()} of {neq.size} elements differ bitwise; first at "
                             f"{i.tolist()}: got {got.ravel()[i]} want {want.ravel()[i]}")


def ulp_distance(a, b):
    """Distance in units in the last place between float32 arrays (NaN == NaN,
    +0 == -0)."""
    a = np.ascontiguousarray(a, np.float32)
    b = np.ascontiguousarray(b, np.float32)
    ia = a.view(np.int32).astype(np.int64)
    ib = b.view(np.int32).astype(np.int64)
    ia = np.where(ia < 0, -(ia & 0x7FFFFFFF), ia)
    ib = np.where(ib < 0, -(ib & 0x7FFFFFFF), ib)
    d = np.abs(ia - ib)
    d = np.where(np.isnan(a) & np.isnan(b), 0, d)
    d = np.where(np.isnan(a) ^ np.isnan(b), 1 << 40, d)
    return d


def oracle_views(O, tensors):
    """OrcViews for HIPTensors sharing one visible shape: raw storage strides,
    view kind, range-nth(0) and the step, as the reference's scheduler reads
    them from tensor-view / tensor-stride."""
    shape = tensors[0].shape
    descs = []
    for t in tensors:
        kind, first, step = [], [], []
        for v in t.views:
            if v.broadcast:
                kind.append(O.KIND_BROADCAST)
            elif v.view is True:
                kind.append(O.KIND_T)
            else:
                kind.append(O.KIND_OTHER)
            first.append(v.range.nth(0))
            step.append(v.range.nth(1) - v.range.nth(0))
        descs.append(dict(stride=list(t.stride), kind=kind, first=first, step=step,
                          offset=t.initial_offset))
    return O.make_views(shape, descs)


class NoBuffer:
    """Stands in for device storage so that view geometry can be exercised on a
    machine without a GPU."""

    def __init__(self, nbytes):
        self.ptr = 0
        self.nbytes = int(nbytes)


def host_tensor(W, shape):
    """A HIPTensor whose storage is never touched (geometry only)."""
    n = int(np.prod(shape, dtype=np.int64))
    return W.HIPTensor(shape, vec=NoBuffer(4 * n))
