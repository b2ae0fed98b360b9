"""Tsitouras 5(4) (mirrors torchode/single_step_methods/tsit5.py)."""
from typing import Optional

from .. import _lib
from ..interpolation import FourthOrderPolynomialInterpolation
from ..terms import ODETerm
from .dopri5 import _LazyTableau
from .runge_kutta import ERKInterpolationData, ExplicitRungeKutta


class Tsit5(ExplicitRungeKutta):
    """7-stage FSAL pair of convergence order 5; ``TABLEAU.b_other`` holds the theta^2..theta^4
    weights of its free quartic dense output."""

    method_id = _lib.TSIT5
    TABLEAU = _LazyTableau(_lib.TSIT5)

    def __init__(self, term: Optional[ODETerm] = None):
        super().__init__(term, Tsit5.TABLEAU)

    def convergence_order(self) -> int:
        return 5

    def build_interpolation(self, data: ERKInterpolationData):
        """reference tsit5.py:123-139"""
        return FourthOrderPolynomialInterpolation.from_erk_step(_lib.TSIT5, data.t0, data.dt, data.y0, data.y1, data.k)
