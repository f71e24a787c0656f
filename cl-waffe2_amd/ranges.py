"""``Range`` -- the index arithmetic behind cl-waffe2 views.

Host-side mirror of ``source/vm/iterator/range.lisp`` for static (integer)
shapes: ``Range`` (:23-27), ``range-size`` (:45-62), ``range-nth`` (:74-98),
``range`` (:109-141) and the composition ``.range`` (:158-263).
"""
from __future__ import annotations

from dataclasses import dataclass
from math import gcd


def _sign(v: int) -> int:
    return (v > 0) - (v < 0)


@dataclass(frozen=True)
class Range:
    """Half-open interval ``[from, to)`` walked with ``step``; a negative step
    walks it from the top (range.lisp:109-126)."""

    start: int
    stop: int
    step: int = 1

    def __post_init__(self):
        if self.step == 0:
            raise ValueError("range: do not create a range whose step is 0")

    @property
    def size(self) -> int:
        """floor(|from - to| / |step|)   (range.lisp:45-62)"""
        return abs(self.start - self.stop) // abs(self.step)

    def nth(self, count: int) -> int:
        """Storage index of the count-th element (range.lisp:74-98)."""
        a, b, c = self.start, self.stop, self.step
        if a > b:
            a, b, c = b, a, -c
        if c < 0:
            a = b + c
        return a + c * count

    def indices(self):
        return [self.nth(i) for i in range(self.size)]


def make_range(start: int, stop: int | None = None, step: int = 1) -> Range:
    """``(range from &optional (to (1+ from)) (step 1))``"""
    if stop is None:
        stop = start + 1
    return Range(start, stop, step)


def compose(new: Range, base: Range | None) -> Range:
    """``(.range new base)``: interpret ``new`` inside the window ``base``
    (range.lisp:158-263)."""
    if base is None:
        return new
    offset = min(base.start, base.stop) if base.step > 0 else max(base.start, base.stop)
    lo = offset + _sign(base.step) * new.start
    hi = offset + _sign(base.step) * new.stop
    step = _sign(new.step) * (abs(base.step * new.step) // gcd(base.step, new.step))
    return Range(min(lo, hi), max(lo, hi), step)
