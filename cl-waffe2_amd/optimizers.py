"""SGD and Adam on HIPTensor parameters.

Mirror of ``source/optimizers/impls/sgd.lisp`` and ``adam.lisp``: an optimiser
object owns one parameter (``defoptimizer`` ties it to ``param``) and
``step(grad)`` is ``step-optimize``.  Two modes:

``nodes``  the reference's composition of element-wise nodes, one launch each
           (``SGD-Compute-Form``, ``Adam-Step-M/V/Param``);
``fused``  one kernel per step (``wf2hip_sgd_step_f32`` / ``wf2hip_adam_step_f32``)
           that performs the same binary32 operations in the same order:
           bit-identical, a few per cent of the memory traffic.
"""
from __future__ import annotations

import ctypes as C
import math

import numpy as np

from . import functional as F
from . import lib as _lib
from .tensor import HIPTensor


def _flat(t: HIPTensor, what: str):
    if not t.is_contiguous():
        raise ValueError(f"{what} must be a contiguous tensor that owns its storage")
    return C.c_void_p(t.ptr), t.size


class SGD:
    """``(SGD param :lr 1e-3)``: ``Param <- Param - Grad * lr``.  Like the
    reference (``(A-=B param (A*=scal grad lr))``, sgd.lisp:24) the gradient is
    scaled in place."""

    def __init__(self, param: HIPTensor, lr: float = 1e-3, mode: str = "fused"):
        self.param, self.lr, self.mode = param, float(np.float32(lr)), mode

    def step(self, grad: HIPTensor) -> HIPTensor:
        if self.mode == "nodes":
            return F.sub_(self.param, F.mul_(grad, self.lr))
        p, n = _flat(self.param, "param")
        g, ng = _flat(grad, "grad")
        if n != ng:
            raise ValueError("param and grad differ in size")
        _lib.check(_lib.get().wf2hip_sgd_step_f32(n, p, g, self.lr))
        return self.param


class Adam:
    """``(Adam param :lr 1e-3 :eps 1e-7 :beta1 0.9 :beta2 0.999)``
    (adam.lisp:4-33).  ``m`` and ``v`` start at zero; ``n`` counts the steps."""

    def __init__(self, param: HIPTensor, lr: float = 1e-3, eps: float = 1e-7, beta1: float = 0.9,
                 beta2: float = 0.999, mode: str = "fused"):
        f32 = lambda x: float(np.float32(x))  # noqa: E731 - the slots are single-float
        self.param, self.mode = param, mode
        self.lr, self.eps, self.beta1, self.beta2 = f32(lr), f32(eps), f32(beta1), f32(beta2)
        self.n = 0
        self.m = HIPTensor(param.shape)
        self.v = HIPTensor(param.shape)

    @staticmethod
    def _expt(base: np.float32, power: int) -> np.float32:
        """``(expt single-float fixnum)``: Common Lisp leaves the algorithm to the
        implementation; this is exponentiation by squaring in single-float products (what
        SBCL does), not a binary64 pow rounded once.  The Lisp glue calls the host's own
        ``expt``, so only this mirror depends on the choice (its last bit is unpinned)."""
        total = base if power & 1 else np.float32(1.0)
        power >>= 1
        while power:
            base = np.float32(base * base)
            if power & 1:
                total = np.float32(base * total)
            power >>= 1
        return total

    def step_lr(self) -> float:
        """``adam-step-lr`` (adam.lisp:78-92) in single-float arithmetic."""
        self.n += 1
        one = np.float32(1.0)
        b1, b2 = np.float32(self.beta1), np.float32(self.beta2)
        num = np.sqrt(one - self._expt(b2, self.n), dtype=np.float32)
        den = one - self._expt(b1, self.n)
        return float(np.float32(self.lr) * (num / den))

    def step(self, grad: HIPTensor) -> HIPTensor:
        lr_t = self.step_lr()
        omb1 = float(np.float32(1.0) - np.float32(self.beta1))   # (!sub 1.0 decay-rate) on host scalars
        omb2 = float(np.float32(1.0) - np.float32(self.beta2))
        if self.mode == "nodes":
            # Adam-Step-M: (A+=B m (!mul (!sub x-grad m) (!sub 1.0 decay-rate)))
            F.add_(self.m, F.mul(F.sub(grad, self.m), omb1))
            # Adam-Step-V: (A+=B v (!mul (!sub 1.0 decay-rate) (!sub (!mul x-grad x-grad) v)))
            F.add_(self.v, F.mul(F.sub(F.mul(grad, grad), self.v), omb2))
            # Adam-Step-Param: (A-=B param (!div (!mul m lr-t) (!add eps (!sqrt v))))
            F.sub_(self.param, F.div(F.mul(self.m, lr_t), F.add(F.sqrt(self.v), self.eps)))
            return self.param
        p, n = _flat(self.param, "param")
        g, ng = _flat(grad, "grad")
        if n != ng:
            raise ValueError("param and grad differ in size")
        _lib.check(_lib.get().wf2hip_adam_step_f32(n, p, g, C.c_void_p(self.m.ptr), C.c_void_p(self.v.ptr),
                                                  omb1, omb2, lr_t, self.eps))
        return self.param
