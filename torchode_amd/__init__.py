"""MI355X-native batch-parallel adaptive Runge-Kutta solver with torchode's API for that path."""

__version__ = "0.1.0"

# the solve loop and its gradients
from .adjoints import AutoDiffAdjoint
from .backsolve import BacksolveAdjoint, JointBacksolveAdjoint

# what a solve is made of: problem, right-hand side, step method, step size controller; what it returns
from .problems import InitialValueProblem
from .terms import ODETerm
from .single_step_methods import Dopri5, Euler, Heun, Tsit5
from .step_size_controllers import FixedStepController, IntegralController, PIDController
from .solution import Solution
from .status_codes import Status

# right-hand sides the whole-solve kernels know, and the benchmark workloads built from them
from . import builtin_terms, workloads
from .builtin_terms import LinearDecay, Lorenz63, MLPField, ReactionDiffusion, VanDerPol

# the one-call interface and its method names (the reference registers these three)
from .interface import register_method, solve_ivp

for _name, _method in (("dopri5", Dopri5), ("tsit5", Tsit5), ("heun", Heun)):
    register_method(_name, _method)
del _name, _method

__all__ = [name for name, value in list(globals().items()) if not name.startswith("_") and (isinstance(value, type) or name in ("solve_ivp", "register_method"))]
