"""MI355X-native batch-parallel adaptive Runge-Kutta solver with torchode's API for that path."""

__version__ = "0.1.0"

from . import builtin_terms, workloads
from .adjoints import AutoDiffAdjoint
from .backsolve import BacksolveAdjoint, JointBacksolveAdjoint
from .builtin_terms import LinearDecay, Lorenz63, MLPField, ReactionDiffusion, VanDerPol
from .problems import InitialValueProblem
from .interface import register_method, solve_ivp
from .single_step_methods import Dopri5, Euler, Heun, Tsit5
from .solution import Solution
from .status_codes import Status
from .step_size_controllers import FixedStepController, IntegralController, PIDController
from .terms import ODETerm

register_method("heun", Heun)
register_method("dopri5", Dopri5)
register_method("tsit5", Tsit5)

__all__ = [
    "AutoDiffAdjoint",
    "BacksolveAdjoint",
    "JointBacksolveAdjoint",
    "InitialValueProblem",
    "register_method",
    "solve_ivp",
    "Dopri5",
    "Euler",
    "Heun",
    "Tsit5",
    "Solution",
    "Status",
    "FixedStepController",
    "IntegralController",
    "PIDController",
    "ODETerm",
    "LinearDecay",
    "VanDerPol",
    "Lorenz63",
    "ReactionDiffusion",
    "MLPField",
]
