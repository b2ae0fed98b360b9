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


def _time_range(t_span, t_eval, batch_size: int):
    """``(t_start, t_end)`` as ``[B]`` each: the given span, else the first and last evaluation time."""
    t_start, t_end = t_span if t_span is not None else (t_eval[:, 0], t_eval[:, -1])
    return _per_sample(t_start, batch_size), _per_sample(t_end, batch_size)


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
    batch_size = y0.shape[0]
    if t_eval is not None and t_eval.ndim == 1:
        t_eval = t_eval.expand((batch_size, -1))
    problem = InitialValueProblem(y0, *_time_range(t_span, t_eval, batch_size), t_eval)

    term = f if isinstance(f, ODETerm) else ODETerm(f, with_args=args is not None)
    if isinstance(method, str):
        method = METHODS[method](term=term)
    if controller is None:
        controller = PIDController(term=term, **DEFAULT_TOLERANCES)
    return AutoDiffAdjoint(method, controller, max_steps=max_steps).solve(problem, term, dt0=dt0, args=args)
