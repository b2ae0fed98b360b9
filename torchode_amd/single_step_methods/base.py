"""Step method protocol (mirrors torchode/single_step_methods/base.py:11-89).

A user-defined step method subclasses ``SingleStepMethod`` and is driven by
``AutoDiffAdjoint.solve`` through exactly these calls.
"""
from typing import Any, Dict, NamedTuple, Optional, Tuple

import torch
import torch.nn as nn

from ..interpolation import LocalInterpolation
from ..problems import InitialValueProblem
from ..terms import ODETerm


class StepResult(NamedTuple):
    y: torch.Tensor
    error_estimate: Optional[torch.Tensor]


class SingleStepMethod(nn.Module):
    def init(self, term: Optional[ODETerm], problem: InitialValueProblem, f0: Optional[torch.Tensor], *, stats: Dict[str, Any], args: Any):
        """State of the method at ``t_start``; ``f0`` is ``f(t_start, y0)`` if the controller already evaluated it."""
        raise NotImplementedError()

    def step(
        self, term: Optional[ODETerm], running: torch.Tensor, y0: torch.Tensor, t0: torch.Tensor, dt: torch.Tensor, state, *,
        stats: Dict[str, Any], args: Any,
    ) -> Tuple[StepResult, Any, Any, Optional[torch.Tensor]]:  # fmt: skip
        """Advance every sample from ``(t0, y0)`` by ``dt``.  Returns the step result (``y1`` and an
        optional error estimate), data for ``build_interpolation``, the next method state and an
        optional int64 ``[B]`` status (``None``: all successful)."""
        raise NotImplementedError()

    def merge_states(self, accept: torch.Tensor, current, previous):
        """Method state that is ``current`` where ``accept`` and ``previous`` elsewhere."""
        raise NotImplementedError()

    def build_interpolation(self, data) -> LocalInterpolation:
        raise NotImplementedError()

    def convergence_order(self) -> int:
        raise NotImplementedError()
