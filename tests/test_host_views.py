"""Host-side view algebra against the reference's own test vectors
(vm/generic-tensor/t/view.lisp:54-69, vm/iterator/test-suites.lisp:14-166,
base-impl/t/apis.lisp:188-221) -- no GPU needed: only geometry is computed."""
import numpy as np
import pytest

from helpers import host_tensor


def elements(t):
    """Storage indices a view visits, row-major (what mref walks)."""
    shape, strides, off = t.geometry()
    idx = np.full(shape, off, dtype=np.int64)
    for ax, (n, s) in enumerate(zip(shape, strides)):
        idx += (np.arange(n) * s).reshape([-1 if i == ax else 1 for i in range(len(shape))])
    return idx.ravel().tolist()


def test_range_size_and_nth(W):
    R = W.make_range
    assert R(0, 10, 1).size == 10 and R(0, 10, 2).size == 5 and R(0, 10, -2).size == 5
    assert R(0, 10, 2).indices() == [0, 2, 4, 6, 8]
    assert R(2, 10, 2).indices() == [2, 4, 6, 8]
    assert R(2, 10, -2).indices() == [8, 6, 4, 2]           # all-dynamic-do-range-test
    assert R(10, 0, -1).indices() == list(range(10))         # from > to flips the step
    assert R(3).indices() == [3]
    with pytest.raises(ValueError):
        R(0, 4, 0)


def test_range_composition(W):
    R, comp = W.make_range, W.compose
    assert comp(R(0, 4, 2), R(2, 10, 2)) == R(2, 6, 2)       # docstring of .range
    assert comp(R(1, 3), R(1, 5)).indices() == [2, 3]
    assert comp(R(1), R(1, 5)).indices() == [2]
    assert comp(R(0, 3), None) == R(0, 3)


def test_view_1d_vectors(W):
    a = host_tensor(W, (10,))
    assert elements(a.view((0, 10, 2))) == [0, 2, 4, 6, 8]
    assert elements(a.view((2, -1, 2)))[:3] == [2, 4, 6]      # (2 9 2): three elements, then 8 by extrapolation
    assert elements(a.view((2, 10, -2))) == [8, 6, 4, 2]
    assert elements(a.view(0)) == [0] and elements(a.view(1)) == [1]
    assert elements(a.view((0, 3))) == [0, 1, 2] and elements(a.view((2, 10)))[0] == 2
    assert elements(a.view((1, 5)).view((1, 3))) == [2, 3]   # slice o slice
    assert elements(a.view((1, 5)).view(1)) == [2]           # slice o index
    assert elements(a.view(1).view(0)) == [1]
    assert a.view((1, 5)).view(True).shape == [10]           # T extends back to the whole axis


def test_broadcast_and_reverser(W):
    o = host_tensor(W, (4, 1))
    b = o.view(True, (":broadcast", 6))
    assert b.shape == [4, 6] and b.geometry()[1] == [1, 0]
    assert b.view(True, True).shape == [4, 1]                # the reverser of !sum
    with pytest.raises(ValueError):
        host_tensor(W, (4, 3)).view(True, (":broadcast", 6))
    with pytest.raises(IndexError):
        host_tensor(W, (4, 3)).view((0, 5))


def test_strides_permute_contiguity(W):
    t = host_tensor(W, (2, 3, 4))
    assert t.stride == [12, 4, 1] and t.is_contiguous()
    p = t.permute(2, 0, 1)
    assert p.shape == [4, 2, 3] and p.geometry()[1] == [1, 12, 4] and not p.is_contiguous()
    assert elements(host_tensor(W, (3, 3)).permute(1, 0)) == [0, 3, 6, 1, 4, 7, 2, 5, 8]
    assert not t.view((0, 1)).is_contiguous()
    with pytest.raises(ValueError):
        t.permute(0, 0, 1)
    with pytest.raises(ValueError):
        W.HIPTensor([1] * 9, vec=object())


def test_dispatch_rules(W):
    """determine-facet-of-nodes: first device in the list with an
    implementation whose reject-p accepts the dtype; otherwise node-not-found
    (defnode.lisp:215-232).  Mirrors the MyBackend test of
    vm/nodes/t/nodes.lisp:12-53."""
    class MyBackend:
        dtype = "float"

    class MyBackendWithImpl(MyBackend):
        pass

    calls = []
    W.define_impl("AddNode", MyBackendWithImpl)(lambda x, y: calls.append("mine") or x)
    with W.with_devices(MyBackend, MyBackendWithImpl, W.HIPTensor):
        assert W.nodes.find_impl("AddNode") is not None
        W.forward("AddNode", MyBackendWithImpl(), MyBackendWithImpl())
        assert calls == ["mine"]                           # MyBackend has no impl: skipped
        assert W.nodes.find_impl("MulNode") is W.nodes.DEVICE_FEATURES[W.HIPTensor]["MulNode"][0]
    with W.with_devices(MyBackend):
        with pytest.raises(W.NodeNotFound):
            W.nodes.find_impl("AddNode")
    assert W.nodes.find_impl("AddNode", dtype="int32") is not None   # arithmetic and moves take every dtype
    with pytest.raises(W.NodeNotFound):                        # the rest reject ints: no device fallback here
        W.nodes.find_impl("ExpNode", dtype="int32")
    with pytest.raises(ValueError):
        W.define_impl("SumNode", W.HIPTensor)                  # cl-waffe2 has no SumNode
    del W.nodes.DEVICE_FEATURES[MyBackendWithImpl]
