"""waffe2-hip: the MI355X (gfx950) tensor-kernel backend for cl-waffe2.

The product is ``libwaffe2-hip.so`` (``csrc/``, C ABI in ``include/waffe2_hip.h``)
plus the Common Lisp glue in ``lisp/``.  This Python package is the host-side
mirror of that glue, used where no Lisp runtime exists: a ``HIPTensor`` class
with cl-waffe2's view algebra, the ``define-impl`` registrations for the
hot-path nodes, and the ``!``-functions composed from them.

Importing the package does not touch the GPU; the first tensor or kernel call
loads the library and initialises device 0.  There is no CPU fallback: without
the built library every operation raises ``HIPExtensionMissing``.
"""
from . import lib
from .lib import HIPError, HIPExtensionMissing
from .ranges import Range, compose, make_range
from .tensor import HIPTensor, Subscript, column_major_strides, parse_view, viewtype
from . import nodes
from .nodes import NodeNotFound, define_impl, forward, with_devices
from . import functional
from . import optimizers
from . import io
from . import nn

__all__ = [
    "lib", "HIPError", "HIPExtensionMissing", "Range", "compose", "make_range", "HIPTensor",
    "Subscript", "column_major_strides", "parse_view", "viewtype", "nodes", "NodeNotFound",
    "define_impl", "forward", "with_devices", "functional",
]
