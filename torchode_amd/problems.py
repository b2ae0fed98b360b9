"""A batch of initial value problems: the container the solvers take (reference torchode/problems.py:6-90)."""
from typing import Optional

import torch


def _agree(what: str, first: torch.Tensor, *others: torch.Tensor) -> bool:
    """All tensors have the same ``dtype`` / ``device`` / batch size as the first."""
    read = (lambda x: x.shape[0]) if what == "batch" else (lambda x: getattr(x, what))
    return all(read(other) == read(first) for other in others)


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

    def __init__(self, y0: torch.Tensor, t_start: Optional[torch.Tensor] = None, t_end: Optional[torch.Tensor] = None,
                 t_eval: Optional[torch.Tensor] = None):  # fmt: skip
        assert t_eval is not None or (t_start is not None and t_end is not None)  # the range comes from t_eval otherwise
        self.y0, self.t_eval = y0, t_eval
        self.t_start = t_eval[:, 0] if t_start is None else t_start
        self.t_end = t_eval[:, -1] if t_end is None else t_end
        self._time_direction = None  # (made when first asked for: four small launches that most solves never need)

        times = (self.t_start, self.t_end) if t_eval is None else (self.t_start, self.t_end, t_eval)
        assert y0.ndim == 2 and self.t_start.ndim == 1 and self.t_end.ndim == 1 and (t_eval is None or t_eval.ndim == 2)
        assert _agree("dtype", *times)
        assert _agree("batch", y0, *times)
        assert _agree("device", y0, *times)

    @property
    def time_direction(self) -> torch.Tensor:
        """``+1`` where ``t_end > t_start``, ``-1`` otherwise (reference problems.py:58-60)."""
        if self._time_direction is None:
            self._time_direction = torch.where(self.t_end > self.t_start, 1, -1)
        return self._time_direction

    # what the solvers ask of a problem
    data_dtype = property(lambda self: self.y0.dtype)
    time_dtype = property(lambda self: self.t_start.dtype)
    device = property(lambda self: self.y0.device)
    batch_size = property(lambda self: self.y0.shape[0])
    n_features = property(lambda self: self.y0.shape[1])
    n_evaluation_points = property(lambda self: 0 if self.t_eval is None else self.t_eval.shape[1])

    def __repr__(self):
        fields = ", ".join(f"{name}={getattr(self, name)}" for name in ("y0", "t_start", "t_end", "t_eval"))
        return f"InitialValueProblem({fields})"
