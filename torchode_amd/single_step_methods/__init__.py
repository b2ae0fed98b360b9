"""Single step methods (mirror torchode/single_step_methods/__init__.py)."""
from .base import SingleStepMethod, StepResult
from .dopri5 import Dopri5
from .euler import Euler
from .heun import Heun
from .runge_kutta import ButcherTableau, ERKInterpolationData, ERKState, ExplicitRungeKutta
from .tsit5 import Tsit5
