"""The two low-order methods of the reference: forward Euler (torchode/single_step_methods/euler.py)
and Heun's method 2(1) (torchode/single_step_methods/heun.py).  The classes here are the operator
path; the per-step kernels know the two methods by ``method_id`` (rows of fewer than 64 features)."""
from typing import Any, Dict, NamedTuple, Optional

import torch

from .. import _lib, differentiable
from ..interpolation import LinearInterpolation, ThirdOrderPolynomialInterpolation
from ..terms import ODETerm
from .base import SingleStepMethod, StepResult
from .runge_kutta import ButcherTableau, ERKInterpolationData, ExplicitRungeKutta


class LinearInterpolationData(NamedTuple):
    t0: torch.Tensor
    dt: torch.Tensor
    y0: torch.Tensor
    y1: torch.Tensor


class Euler(SingleStepMethod):
    """``y1 = y0 + dt f(t0, y0)``, no error estimate (a controller then keeps the step size), linear
    dense output."""

    method_id = _lib.EULER

    def __init__(self, term: Optional[ODETerm] = None):
        super().__init__()
        self.term = term

    def init(self, term, problem, f0, *, stats: Dict[str, Any], args: Any):
        return None

    def step(self, term, running, y0, t0, dt, state, *, stats, args):
        term_ = term if term is not None else self.term
        assert term_ is not None
        _lib.require_device(y0, t0, dt)
        y0, dt = y0.contiguous(), dt.contiguous()
        B, F = y0.shape
        k = term_.vf(t0, y0, stats, args).to(y0.dtype).contiguous()

        def kernel():
            y1 = torch.empty_like(y0)
            one = (_lib.C.c_double * 1)(1.0)
            rc = _lib.load().tode_erk_stage(
                _lib.dtype_code(y0.dtype, dt.dtype), B, F, 1, one, 0.0, None, _lib.ptr(dt), _lib.ptr(y0), _lib.ptr(k), _lib.ptr(y1), None,
                _lib.stream_of(y0),
            )  # fmt: skip
            _lib.check(rc, "tode_erk_stage")
            return y1

        y1 = differentiable.through(kernel, lambda dt_, y0_, k_: differentiable.stage([1.0], 0.0, None, dt_, y0_, k_), dt, y0, k)
        return StepResult(y1, None), LinearInterpolationData(t0, dt, y0, y1), state, None

    def merge_states(self, accept, current, previous):
        return None

    def convergence_order(self) -> int:
        return 1

    def build_interpolation(self, data: LinearInterpolationData):
        return LinearInterpolation(data.t0, data.dt, data.y0, data.y1)


# Heun 2(1): the trapezoidal rule as the result, the Euler step as the embedded low-order solution.
_HEUN_NODES = [0.0, 1.0]
_HEUN_STAGES = [[], [1.0]]
_HEUN_WEIGHTS, _HEUN_EULER_WEIGHTS = [0.5, 0.5], [1.0, 0.0]


class Heun(ExplicitRungeKutta):
    """Two stages, error estimate against the Euler step, Hermite cubic dense output (stage and sum
    kernels with this tableau)."""

    method_id = _lib.HEUN
    TABLEAU = ButcherTableau.from_lists(c=_HEUN_NODES, a=_HEUN_STAGES, b=_HEUN_WEIGHTS, b_low_order=_HEUN_EULER_WEIGHTS)

    def __init__(self, term: Optional[ODETerm] = None):
        super().__init__(term, type(self).TABLEAU)

    def convergence_order(self) -> int:
        return 2

    def build_interpolation(self, data: ERKInterpolationData):
        first_and_last_slopes = data.k
        return ThirdOrderPolynomialInterpolation.from_k(data.t0, data.dt, data.y0, data.y1, first_and_last_slopes)
