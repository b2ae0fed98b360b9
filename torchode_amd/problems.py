"""Batch of initial value problems (mirrors torchode/problems.py:6-90)."""
from typing import Optional

import torch


def _same(attr, *tensors):
    return all(getattr(a, attr) == getattr(b, attr) for a, b in zip(tensors[:-1], tensors[1:]))


class InitialValueProblem:
    """``B`` independent problems ``dy/dt = f(t, y)``, ``y(t_start) = y0``.

    ``y0`` is ``[B, F]``; ``t_start``/``t_end`` are ``[B]`` and ``t_eval`` is ``[B, E]``
    in one time dtype that may differ from the data dtype.  Missing ``t_start`` /
    ``t_end`` default to the first / last column of ``t_eval``.  Each sample may run
    forwards or backwards in time (``time_direction`` is ``+1`` where
    ``t_end > t_start`` and ``-1`` otherwise).  Without ``t_eval`` the solution is
    reported at ``t_end`` only.  Shape, dtype and device mismatches are assertion
    errors, as in the reference (problems.py:44-56).
    """

    def __init__(
        self,
        y0: torch.Tensor,
        t_start: Optional[torch.Tensor] = None,
        t_end: Optional[torch.Tensor] = None,
        t_eval: Optional[torch.Tensor] = None,
    ):
        self.y0 = y0
        self.t_eval = t_eval
        if t_start is None:
            assert t_eval is not None
            t_start = t_eval[:, 0]
        if t_end is None:
            assert t_eval is not None
            t_end = t_eval[:, -1]
        self.t_start = t_start
        self.t_end = t_end
        self.time_direction = torch.where(self.t_end > self.t_start, 1, -1)

        assert y0.ndim == 2
        assert self.t_start.ndim == 1 and self.t_end.ndim == 1
        assert _same("dtype", self.t_start, self.t_end)
        assert y0.shape[0] == self.t_start.shape[0] == self.t_end.shape[0]
        assert _same("device", y0, self.t_start, self.t_end)
        if t_eval is not None:
            assert t_eval.ndim == 2
            assert _same("dtype", self.t_start, t_eval)
            assert self.t_start.shape[0] == t_eval.shape[0]
            assert _same("device", self.t_start, t_eval)

    @property
    def data_dtype(self):
        return self.y0.dtype

    @property
    def time_dtype(self):
        return self.t_start.dtype

    @property
    def device(self):
        return self.y0.device

    @property
    def batch_size(self):
        return self.y0.shape[0]

    @property
    def n_features(self):
        return self.y0.shape[1]

    @property
    def n_evaluation_points(self):
        return 0 if self.t_eval is None else self.t_eval.shape[1]

    def __repr__(self):
        return (
            f"InitialValueProblem(y0={self.y0}, t_start={self.t_start}, "
            f"t_end={self.t_end}, t_eval={self.t_eval})"
        )
