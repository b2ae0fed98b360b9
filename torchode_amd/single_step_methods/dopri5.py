"""Dormand-Prince 5(4) (mirrors torchode/single_step_methods/dopri5.py)."""
from typing import Optional

from .. import _lib
from ..interpolation import FourthOrderPolynomialInterpolation
from ..terms import ODETerm
from .runge_kutta import ERKInterpolationData, ExplicitRungeKutta, library_tableau


class _LazyTableau:
    """Class attribute ``TABLEAU``: read from the kernel library on first use."""

    def __init__(self, method_id):
        self.method_id, self.value = method_id, None

    def __get__(self, obj, owner):
        if self.value is None:
            self.value = library_tableau(self.method_id)
        return self.value


class Dopri5(ExplicitRungeKutta):
    """7-stage FSAL pair of convergence order 5 with a quartic dense output through the step's mid point."""

    method_id = _lib.DOPRI5
    TABLEAU = _LazyTableau(_lib.DOPRI5)

    def __init__(self, term: Optional[ODETerm] = None):
        super().__init__(term, Dopri5.TABLEAU)

    def convergence_order(self) -> int:
        return 5

    def build_interpolation(self, data: ERKInterpolationData):
        """reference dopri5.py:53-60"""
        return FourthOrderPolynomialInterpolation.from_erk_step(_lib.DOPRI5, data.t0, data.dt, data.y0, data.y1, data.k)
