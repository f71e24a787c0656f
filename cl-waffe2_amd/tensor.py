"""``HIPTensor`` -- the device tensor class of the backend.

Host-side mirror (static shapes, fp32) of the parts of cl-waffe2's
``AbstractTensor`` protocol a backend has to supply
(``source/vm/generic-tensor/tensor.lisp:40-210``):

* allocation when the facet is ``:exist`` -- zero-filled, like
  ``make-array :initial-element 0`` in ``backends/lisp/tensor.lisp:12-28``;
* ``tensor-vec`` holding an opaque device buffer, released by the finalizer
  (``tensor.lisp:323-329``);
* ``vref`` / ``(setf vref)`` (``tensor.lisp:719-746``) -- one element across
  PCIe, for tests and ``Mat->ScalarNode`` only;
* views: ``view`` (``tensor.lisp:820-864``), ``parse-view`` / ``Subscript``
  (``view.lisp:71-206``), strides for ``:column`` (C-contiguous) order
  (``utils.lisp:50-67``), ``permute*`` (``tensor.lisp:936-991``).

The kernels never see this class: ``geometry()`` flattens a view into the
(shape, effective stride, start offset) triple that ``wf2hip_view2`` carries.
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass
from typing import Sequence

import math

import numpy as np

from . import lib as _lib
from .ranges import Range, compose, make_range


class DeviceBuffer:
    """Zero-initialised device memory owned by one or more tensors."""

    def __init__(self, nbytes: int, zero: bool = True):
        self.nbytes = int(nbytes)
        p = C.c_void_p()
        alloc = _lib.get().wf2hip_malloc if zero else _lib.get().wf2hip_malloc_uninitialized
        _lib.check(alloc(C.byref(p), self.nbytes))
        self.ptr = p.value or 0

    def __del__(self):  # tensor-finalizer
        try:
            if self.ptr and _lib._lib is not None:
                _lib._lib.wf2hip_free(C.c_void_p(self.ptr))
                self.ptr = 0
        except Exception:
            pass


@dataclass(frozen=True)
class Subscript:
    """One axis of a view (``view.lisp:71-75``): the syntax that produced it,
    whether it is a ``(:broadcast n)`` axis, and its Range over the storage."""

    view: object
    broadcast: bool
    range: Range
    repeat: int = 1  # n of (:broadcast n)


def viewtype(view) -> str:
    """``view.lisp:120-138``"""
    if isinstance(view, (tuple, list)):
        if len(view) == 2 and view[0] in (":broadcast", ":index"):
            return view[0][1:]
        if len(view) == 2:
            return "slice"
        if len(view) == 3:
            return "slice-step"
        raise ValueError(f"Cannot parse a view {view!r}: it should be (start stop) or (start stop step)")
    if isinstance(view, Range):
        return "range"
    if view is True:
        return "t"
    if isinstance(view, (int, np.integer)):
        return "index"
    raise ValueError(f"Unknown view {view!r}")


def _absolute(size: int, v: int) -> int:
    return size + v if v < 0 else v


def parse_view(base_size: int, past: Subscript | None, view) -> Subscript:
    """``parse-view`` (``view.lisp:169-206``) for one axis."""
    kind = viewtype(view)
    viewed = past.range.size if past is not None else base_size
    if kind == "t":
        # T extends the previous view back to the whole axis; over a broadcast
        # axis it gives the size-1 axis underneath (the `reverser` of !sum).
        if past is not None and past.broadcast:
            return Subscript(past.view, False, past.range)
        return Subscript(True, False, make_range(0, base_size))
    if kind == "broadcast":
        n = int(view[1])
        if viewed != 1:
            raise ValueError(f"(:broadcast {n}) needs an axis of size 1, got {viewed}")
        base = past.range if past is not None else None
        return Subscript((":broadcast", n), True, compose(make_range(0), base), n)
    if kind == "index":
        idx = view[1] if isinstance(view, (tuple, list)) else view
        idx = _absolute(viewed, int(idx))
        new = make_range(idx)
    elif kind == "slice":
        new = make_range(_absolute(viewed, int(view[0])), _absolute(viewed, int(view[1])))
    elif kind == "slice-step":
        new = make_range(_absolute(viewed, int(view[0])), _absolute(viewed, int(view[1])), int(view[2]))
    else:
        new = view
    lo, hi = min(new.start, new.stop), max(new.start, new.stop)
    if lo < 0 or hi > viewed:
        raise IndexError(f"view {view!r} is outside an axis of size {viewed}")
    base = past.range if (past is not None and past.view is not True) else None
    return Subscript(view, False, compose(new, base))


def column_major_strides(shape: Sequence[int]) -> list[int]:
    """Strides of cl-waffe2's default ``:column`` order = C-contiguous
    (``utils.lisp:50-67``)."""
    strides, acc = [], 1
    for s in reversed(shape):
        strides.append(acc)
        acc *= int(s)
    return strides[::-1]


# cl-waffe2's dtype keyword -> numpy type of the host copy
# (``dtype->lisp-type``, ``source/vm/generic-tensor/dtype.lisp``)
DTYPES = {"float": np.float32, "double": np.float64, "int32": np.int32, "uint32": np.uint32,
          "int16": np.int16, "uint16": np.uint16, "int8": np.int8, "uint8": np.uint8}


ITEMSIZE = {name: np.dtype(t).itemsize for name, t in DTYPES.items()}


class HIPTensor:
    """A tensor on the GPU, possibly a view of another one's storage.  Every node
    of the path runs on :float; the other dtypes have the arithmetic / move
    nodes only (and :uint32 receives ArgMax-Node / ArgMin-Node results)."""

    def __init__(self, shape: Sequence[int], *, vec: DeviceBuffer | None = None,
                 strides: Sequence[int] | None = None, views: Sequence[Subscript] | None = None,
                 offset: int = 0, initial_element: float | None = 0.0, dtype: str = "float"):
        if dtype not in DTYPES:
            raise ValueError(f"HIPTensor has no dtype {dtype}; known: {sorted(DTYPES)}")
        self.dtype = dtype
        self.itemsize = ITEMSIZE[dtype]
        self.orig_shape = [int(s) for s in shape]
        if len(self.orig_shape) < 1 or len(self.orig_shape) > _lib.MAX_RANK:
            raise ValueError(f"HIPTensor rank must be 1..{_lib.MAX_RANK}")
        if any(s < 0 for s in self.orig_shape):
            raise ValueError("negative extent")
        self.stride = list(strides) if strides is not None else column_major_strides(self.orig_shape)
        # full views are built on first use: most tensors are temporaries that are never viewed
        self._views = list(views) if views is not None else None
        self.initial_offset = int(offset)
        # (shape, strides, offset), computed once: a tensor's views never change
        self._geometry = None if views is not None else (tuple(self.orig_shape), tuple(self.stride), self.initial_offset)
        self._contiguous = None
        if vec is None:
            n = math.prod(self.orig_shape)
            # initial_element None = an InputTensor temporary (make-input): its
            # first use overwrites it, so it is not zero-filled
            vec = DeviceBuffer(self.itemsize * n, zero=initial_element is not None and initial_element == 0)
            if initial_element and n:
                if dtype == "float":
                    _lib.check(_lib.get().wf2hip_fill_f32(C.c_void_p(vec.ptr), n, float(initial_element)))
                else:
                    host = np.full(n, initial_element, DTYPES[dtype])
                    _lib.check(_lib.get().wf2hip_memcpy_h2d(C.c_void_p(vec.ptr), host.ctypes.data_as(C.c_void_p),
                                                           host.nbytes))
        self.vec = vec

    # -- geometry -----------------------------------------------------------
    @property
    def shape(self) -> list[int]:
        """Visible shape (``compute-visible-shape``, ``view.lisp:216-221``)."""
        return list(self._geom()[0])

    @property
    def views(self) -> list:
        if self._views is None:
            self._views = [Subscript(True, False, make_range(0, s)) for s in self.orig_shape]
        return self._views

    @property
    def ndim(self) -> int:
        return len(self.orig_shape)

    @property
    def size(self) -> int:
        n = 1
        for extent in self._geom()[0]:
            n *= extent
        return n

    def geometry(self):
        """(shape, effective strides, start offset) in elements: what
        call-with-view computes per axis as stride x step and
        initial-offset + stride x range-nth(view, 0)
        (``call-with-view.lisp:120-137,168-195``)."""
        shape, strides, off = self._geom()
        return list(shape), list(strides), off

    def _geom(self):
        if self._geometry is None:
            shape, strides, off = [], [], self.initial_offset
            for v, st in zip(self.views, self.stride):
                if v.broadcast:
                    shape.append(v.repeat)
                    strides.append(0)
                    off += st * v.range.nth(0)
                else:
                    shape.append(v.range.size)
                    strides.append(st * (v.range.nth(1) - v.range.nth(0)))
                    off += st * v.range.nth(0)
            self._geometry = (tuple(shape), tuple(strides), off)
        return self._geometry

    def is_contiguous(self) -> bool:
        if self._contiguous is None:
            shape, strides, off = self._geom()
            self._contiguous = off == 0 and list(strides) == column_major_strides(shape) and \
                math.prod(shape) * self.itemsize == self.vec.nbytes
        return self._contiguous

    @property
    def ptr(self) -> int:
        return self.vec.ptr

    # -- construction ---------------------------------------------------------
    @classmethod
    def from_numpy(cls, array, dtype: str = "float") -> "HIPTensor":
        a = np.ascontiguousarray(array, dtype=DTYPES[dtype])
        t = cls(a.shape if a.ndim else (1,), initial_element=None, dtype=dtype)
        if a.size:
            _lib.check(_lib.get().wf2hip_memcpy_h2d(C.c_void_p(t.vec.ptr), a.ctypes.data_as(C.c_void_p), a.nbytes))
        return t

    def storage_numpy(self) -> np.ndarray:
        """The whole underlying storage, flat."""
        n = self.vec.nbytes // self.itemsize
        out = np.empty(n, DTYPES[self.dtype])
        if n:
            _lib.check(_lib.get().wf2hip_memcpy_d2h(out.ctypes.data_as(C.c_void_p), C.c_void_p(self.vec.ptr),
                                                   self.itemsize * n))
        return out

    def numpy(self) -> np.ndarray:
        """The visible tensor as a host array (bulk transfer + host-side
        indexing; the analogue of ``convert-tensor-facet`` to a simple-array,
        ``source/array-converter.lisp:93-151``)."""
        flat = self.storage_numpy()
        shape, strides, off = self.geometry()
        if any(s == 0 for s in shape):
            return np.empty(shape, DTYPES[self.dtype])
        idx = np.full(shape, off, dtype=np.int64)
        for ax, (n, st) in enumerate(zip(shape, strides)):
            ix = np.arange(n, dtype=np.int64) * st
            idx += ix.reshape([-1 if i == ax else 1 for i in range(len(shape))])
        return flat[idx]

    # -- element access -------------------------------------------------------
    def vref(self, index: int) -> float:
        """Element ``index`` of the storage (``tensor.lisp:719-733``)."""
        out = np.empty(1, DTYPES[self.dtype])
        _lib.check(_lib.get().wf2hip_memcpy_d2h(out.ctypes.data_as(C.c_void_p),
                                               C.c_void_p(self.vec.ptr + self.itemsize * int(index)), self.itemsize))
        return out[0].item()

    def set_vref(self, index: int, value: float) -> None:
        v = np.asarray([value], DTYPES[self.dtype])
        _lib.check(_lib.get().wf2hip_memcpy_h2d(C.c_void_p(self.vec.ptr + self.itemsize * int(index)),
                                               v.ctypes.data_as(C.c_void_p), self.itemsize))

    # -- views ------------------------------------------------------------------
    def view(self, *subscripts) -> "HIPTensor":
        """``(view tensor &rest subscripts)``; missing trailing subscripts are T."""
        if len(subscripts) > self.ndim:
            raise ValueError(f"view: {len(subscripts)} subscripts for a rank-{self.ndim} tensor")
        subs = list(subscripts) + [True] * (self.ndim - len(subscripts))
        new = [parse_view(base, past, s) for base, past, s in zip(self.orig_shape, self.views, subs)]
        return HIPTensor(self.orig_shape, vec=self.vec, strides=self.stride, views=new,
                         offset=self.initial_offset, dtype=self.dtype)

    def permute(self, *order: int) -> "HIPTensor":
        """Zero-copy axis permutation; ``order[i]`` is the current axis that
        becomes axis ``i`` (``permute*`` reorders shape/stride/view alike,
        ``tensor.lisp:936-991``)."""
        if sorted(order) != list(range(self.ndim)):
            raise ValueError(f"permute: {order} is not a permutation of 0..{self.ndim - 1}")
        return HIPTensor([self.orig_shape[i] for i in order], vec=self.vec,
                         strides=[self.stride[i] for i in order],
                         views=[self.views[i] for i in order], offset=self.initial_offset,
                         dtype=self.dtype)

    def __repr__(self):
        return f"<HIPTensor {self.shape} views={[v.view for v in self.views]}>"
