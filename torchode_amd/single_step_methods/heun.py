"""Heun's method, 2(1) (mirrors torchode/single_step_methods/heun.py)."""
from typing import Optional

from ..interpolation import ThirdOrderPolynomialInterpolation
from ..terms import ODETerm
from .runge_kutta import ButcherTableau, ERKInterpolationData, ExplicitRungeKutta


class Heun(ExplicitRungeKutta):
    """Two stages, error estimate against the Euler step, Hermite cubic dense output.  Runs through
    the protocol path (stage and sum kernels with this tableau)."""

    TABLEAU = ButcherTableau.from_lists(c=[0.0, 1.0], a=[[], [1.0]], b=[1 / 2, 1 / 2], b_low_order=[1.0, 0.0])

    def __init__(self, term: Optional[ODETerm] = None):
        super().__init__(term, Heun.TABLEAU)

    def convergence_order(self) -> int:
        return 2

    def build_interpolation(self, data: ERKInterpolationData):
        return ThirdOrderPolynomialInterpolation.from_k(data.t0, data.dt, data.y0, data.y1, data.k)
