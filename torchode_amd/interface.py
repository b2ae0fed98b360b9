"""One call from a right-hand side to a solution (reference torchode/interface.py:17-97)."""
from typing import Any, Callable, Dict, Optional, Tuple, Union

import torch

from .adjoints import AutoDiffAdjoint
from .problems import InitialValueProblem
from .single_step_methods import SingleStepMethod
from .solution import Solution
from .step_size_controllers import PIDController, StepSizeController
from .terms import ODETerm

METHODS: Dict[str, Callable[..., SingleStepMethod]] = {}
DEFAULT_TOLERANCES = dict(atol=1e-7, rtol=1e-7, pcoeff=0.2, icoeff=0.5, dcoeff=0.0)  # interface.py:79-81


def register_method(name: str, constructor: Callable[[ODETerm], SingleStepMethod]):
    """Make ``solve_ivp(..., method=name)`` construct the step method with ``constructor(term=term)``."""
    METHODS[name] = constructor


def _per_sample(t: torch.Tensor, batch_size: int) -> torch.Tensor:
    """A scalar time shared by the batch, as ``[B]``."""
    return t.expand(batch_size) if t.ndim == 0 else t


def solve_ivp(
    f: Union[ODETerm, Callable],
    y0: torch.Tensor,
    t_eval: Optional[torch.Tensor],
    *,
    t_span: Optional[Tuple[torch.Tensor, torch.Tensor]] = None,
    method: Union[str, SingleStepMethod] = "tsit5",
    max_steps: Optional[int] = None,
    controller: Optional[StepSizeController] = None,
    dt0: Optional[torch.Tensor] = None,
    args: Any = None,
) -> Solution:
    """Solve a batch of initial value problems (reference interface.py:21-97).

    ``f`` is an ``ODETerm`` or a callable ``f(t, y)`` (``f(t, y, args)`` when ``args`` is given);
    ``t_eval`` is ``[B, E]`` or ``[E]`` (shared by the batch); ``t_span`` defaults to the first and
    last evaluation time; ``method`` is a registered name or a step method object; the default
    controller is ``PIDController(atol=1e-7, rtol=1e-7, pcoeff=0.2, icoeff=0.5, dcoeff=0.0)``."""
    term = f if isinstance(f, ODETerm) else ODETerm(f, with_args=args is not None)
    step_method = method if isinstance(method, SingleStepMethod) else METHODS[method](term=term)
    step_size_controller = controller if controller is not None else PIDController(term=term, **DEFAULT_TOLERANCES)

    batch_size = y0.shape[0]
    if t_eval is not None and t_eval.ndim == 1:
        t_eval = t_eval.expand((batch_size, -1))
    t_start, t_end = t_span if t_span is not None else (t_eval[:, 0], t_eval[:, -1])
    problem = InitialValueProblem(y0, _per_sample(t_start, batch_size), _per_sample(t_end, batch_size), t_eval)
    solver = AutoDiffAdjoint(step_method, step_size_controller, max_steps=max_steps)
    return solver.solve(problem, term, dt0=dt0, args=args)
