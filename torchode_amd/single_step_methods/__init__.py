"""Single step methods: the protocol, the explicit Runge-Kutta machinery and the reference's four methods."""
from .base import SingleStepMethod, StepResult
from .runge_kutta import ButcherTableau, ERKInterpolationData, ERKState, ExplicitRungeKutta
from .fifth_order import Dopri5, Tsit5
from .low_order import Euler, Heun

__all__ = ["SingleStepMethod", "StepResult", "ButcherTableau", "ERKInterpolationData", "ERKState", "ExplicitRungeKutta", "Dopri5", "Tsit5", "Euler", "Heun"]
