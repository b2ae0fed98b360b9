"""One-call interface (mirrors torchode/interface.py)."""
from typing import Any, Callable, Optional, Tuple, Union

import torch

from .adjoints import AutoDiffAdjoint
from .problems import InitialValueProblem
from .single_step_methods import SingleStepMethod
from .solution import Solution
from .step_size_controllers import PIDController, StepSizeController
from .terms import ODETerm

METHODS = {}


def register_method(name: str, constructor: Callable[[ODETerm], SingleStepMethod]):
    """Make ``solve_ivp(..., method=name)`` construct the step method with ``constructor(term=term)``."""
    METHODS[name] = constructor


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
    if isinstance(f, ODETerm):
        term = f
    else:
        term = ODETerm(f, with_args=True) if args is not None else ODETerm(f)
    if not isinstance(method, SingleStepMethod):
        method = METHODS[method](term=term)
    if controller is None:
        controller = PIDController(term=term, atol=1e-7, rtol=1e-7, pcoeff=0.2, icoeff=0.5, dcoeff=0.0)
    adjoint = AutoDiffAdjoint(method, controller, max_steps=max_steps)

    batch_size = y0.shape[0]
    if t_eval is not None and t_eval.ndim == 1:
        t_eval = t_eval.expand((batch_size, -1))
    if t_span is not None:
        t_start, t_end = t_span
    else:
        t_start, t_end = t_eval[:, 0], t_eval[:, -1]
    if t_start.ndim == 0:
        t_start = t_start.expand(batch_size)
    if t_end.ndim == 0:
        t_end = t_end.expand(batch_size)
    problem = InitialValueProblem(y0, t_start, t_end, t_eval)
    return adjoint.solve(problem, term, dt0=dt0, args=args)
