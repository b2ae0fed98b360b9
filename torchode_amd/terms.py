"""ODE term wrapper (mirrors torchode/terms.py:9-63)."""
from typing import Any, Callable, Dict

import torch
import torch.nn as nn

from .problems import InitialValueProblem


class ODETerm(nn.Module):
    """``dy/dt = f(t, y)`` (or ``f(t, y, args)`` with ``with_args=True``).

    With ``with_stats=True`` (default) the solve reports ``stats["n_f_evals"]``, an
    int64 ``[B]`` tensor **on the CPU** that counts evaluations of ``f`` on the whole
    batch (every sample carries the same count).  ``f`` may be one of the modules in
    ``torchode_amd.builtin_terms``; the solver then evaluates it inside the
    persistent kernel and never calls it from Python.
    """

    def __init__(self, f: Callable, *, with_stats: bool = True, with_args: bool = False):
        super().__init__()
        self.f = f
        self.with_stats = with_stats
        self.with_args = with_args

    def init(self, problem: InitialValueProblem, stats: Dict[str, Any]):
        if not self.with_stats:
            return
        stats["n_f_evals"] = torch.zeros(problem.batch_size, device="cpu", dtype=torch.long)

    def vf(self, t, y, stats: Dict[str, Any], args: Any):
        """Evaluate the vector field once on the whole batch."""
        if self.with_stats:
            stats["n_f_evals"].add_(1)
        if self.with_args:
            return self.f(t, y, args)
        return self.f(t, y)
