"""The two embedded 5(4) pairs whose coefficients live in the kernel library: Dormand-Prince and Tsitouras.

Both are 7-stage, first-same-as-last pairs with a quartic dense output; the whole-solve and per-step
kernels know them by ``method_id``, and the operator path reads the same coefficients back from the
library (``library_tableau``), so every path steps with identical numbers.  Reference:
torchode/single_step_methods/dopri5.py:11-60 and tsit5.py:74-139.
"""
from typing import Optional

from .. import _lib
from ..interpolation import FourthOrderPolynomialInterpolation
from ..terms import ODETerm
from .runge_kutta import ERKInterpolationData, ExplicitRungeKutta, library_tableau


class _LibraryTableau:
    """Descriptor behind ``TABLEAU``: asks the kernel library on first access, then keeps the answer."""

    def __init__(self, method_id: int):
        self.method_id = method_id
        self.cached = None

    def __get__(self, instance, owner):
        if self.cached is None:
            self.cached = library_tableau(self.method_id)
        return self.cached


def _dense_output(method_id: int):
    """``build_interpolation`` of a pair: one kernel from the step's seven slopes to the five quartic
    coefficients, with the pair's own dense-output weights (reference dopri5.py:53-60 through the step's
    mid point, tsit5.py:123-139 through ``b_other``).  It does not look at ``self``, so it can be called
    on the class as well."""

    def build_interpolation(self, data: ERKInterpolationData):
        return FourthOrderPolynomialInterpolation.from_erk_step(method_id, data.t0, data.dt, data.y0, data.y1, data.k)

    return build_interpolation


class _LibraryPair(ExplicitRungeKutta):
    def __init__(self, term: Optional[ODETerm] = None):
        super().__init__(term, type(self).TABLEAU)

    def convergence_order(self) -> int:
        return 5


class Dopri5(_LibraryPair):
    """Dormand-Prince 5(4)."""

    method_id = _lib.DOPRI5
    TABLEAU = _LibraryTableau(_lib.DOPRI5)
    build_interpolation = _dense_output(_lib.DOPRI5)


class Tsit5(_LibraryPair):
    """Tsitouras 5(4); ``TABLEAU.b_other`` holds the theta^2..theta^4 weights of its free dense output."""

    method_id = _lib.TSIT5
    TABLEAU = _LibraryTableau(_lib.TSIT5)
    build_interpolation = _dense_output(_lib.TSIT5)
