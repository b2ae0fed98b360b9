"""Gradients through the operator kernels of the protocol path.

The reference's loop is torch operations throughout (torchode/adjoints.py:135-260), so autograd
reaches every input through any mix of the library's and a user's step methods, controllers and
interpolants.  Here the library's own protocol methods run HIP kernels, which autograd does not see.
``through(kernel, formula, *inputs)`` closes that gap one operator at a time: the values come from
the kernel, as without gradients (same bits), and when an input requires grad the result carries a
graph node whose backward pass evaluates ``formula`` -- the operator written as the torch operations
the reference issues at that place -- on the saved inputs and lets autograd differentiate it.
Whatever a user's plug-in does between the operators is recorded by autograd as written.

The formulas below follow the reference's choice of operations where the derivative depends on it
(``torch.maximum`` halves a cotangent at a tie where ``clamp`` hands it on, ``torch.where`` feeds
both branches).
"""
from math import sqrt
from typing import Callable, Optional, Sequence

import torch
from torch.autograd.function import once_differentiable


class _KernelThenFormula(torch.autograd.Function):
    @staticmethod
    def forward(ctx, kernel: Callable, formula: Callable, *inputs):
        outs = kernel()
        single = isinstance(outs, torch.Tensor)
        outs = (outs,) if single else tuple(outs)
        ctx.formula, ctx.inputs = formula, inputs
        ctx.mark_non_differentiable(*[o for o in outs if not o.is_floating_point()])
        ctx.set_materialize_grads(False)
        return outs[0] if single else outs

    @staticmethod
    @once_differentiable
    def backward(ctx, *grads):
        needs = ctx.needs_input_grad[2:]
        live = []
        for x, need in zip(ctx.inputs, needs):
            if isinstance(x, torch.Tensor):
                x = x.detach()
                if need:
                    x = x.requires_grad_()
            live.append(x)
        with torch.enable_grad():
            outs = ctx.formula(*live)
            outs = (outs,) if isinstance(outs, torch.Tensor) or outs is None else tuple(outs)
            targets, cotangents = [], []
            for out, grad in zip(outs, grads):
                if out is not None and grad is not None and out.requires_grad:
                    targets.append(out)
                    cotangents.append(grad if grad.dtype == out.dtype else grad.to(out.dtype))
            wrt = [x for x, need in zip(live, needs) if need]
            found = iter(torch.autograd.grad(targets, wrt, cotangents, allow_unused=True) if targets and wrt else [None] * len(wrt))
        return (None, None, *[next(found) if need else None for need in needs])


def tracked(*tensors) -> bool:
    """True if a result computed from ``tensors`` has to carry a graph."""
    return torch.is_grad_enabled() and any(isinstance(x, torch.Tensor) and x.requires_grad for x in tensors)


def through(kernel: Callable, formula: Callable, *inputs):
    """``kernel()``: a closure that launches a library kernel on the values of ``inputs`` and returns its result
    tensors.  ``formula(*inputs)``: the same results (``None`` for those that carry no gradient: masks, status
    codes) as differentiable torch operations.  The formula is only ever evaluated in a backward pass."""
    if not tracked(*inputs):
        return kernel()
    return _KernelThenFormula.apply(kernel, formula, *inputs)


# ----------------------------------------------------------------------------------------------------
# The operators as torch operations.  Constants (tableau rows, tolerances, exponents) are bound by the
# caller; tensor arguments are the operator's differentiable inputs.
# ----------------------------------------------------------------------------------------------------


def _weighted_sum(weights: Sequence[float], ks: Sequence[torch.Tensor]):
    total = None
    for w, k in zip(weights, ks):
        if w != 0.0:
            total = w * k if total is None else total + w * k
    return total


def stage(a_row: Sequence[float], c: float, t0: Optional[torch.Tensor], dt, y0, *ks):
    """reference runge_kutta.py:259-262: ``y_i = y0 + dt sum_j a_ij k_j``, ``t_i = t0 + c_i dt``."""
    s = _weighted_sum(a_row, ks)
    y_i = y0 if s is None else y0 + dt.to(y0.dtype)[:, None] * s
    return y_i if t0 is None else (y_i, t0 + c * dt)


def combine(weights: Sequence[float], dt, base: Optional[torch.Tensor], *ks):
    """reference runge_kutta.py:265-269: ``base + sum_s (dt w_s) k_s``."""
    s = _weighted_sum(weights, ks)
    s = torch.zeros_like(ks[0]) if s is None else dt.to(ks[0].dtype)[:, None] * s
    return s if base is None else base + s


def select_rows(mask: torch.Tensor, current, previous):
    m = mask.view(torch.bool) if mask.dtype == torch.uint8 else mask
    return torch.where(m[:, None] if current.ndim == 2 else m, current, previous)


def rms(x):
    return torch.linalg.vector_norm(x / sqrt(x.shape[1]), ord=2, dim=1)


def maximum_norm(x):
    return torch.linalg.vector_norm(x, ord=torch.inf, dim=1)


def error_scale(atol: float, rtol: float, y0, y1, err):
    """reference step_size_controllers.py:393-397: the error estimate over its bounds."""
    return err.abs() / (atol + rtol * torch.maximum(y0.abs(), y1.abs()))


def tolerance_scale(atol: float, rtol: float, y_ref, v):
    return v * torch.reciprocal(atol + rtol * y_ref.abs())


def decide(p: dict, accept: torch.Tensor, dt, norm_or_none, y0, y1, err, prev, pprev):
    """reference step_size_controllers.py:393-429 / 738-774 with ``dt_factor`` (:289-294, 598-620) and
    ``update_state`` (:640-671).  ``p``: tolerances, norm, exponents, limits; ``accept``: the kernel's decision.
    Returns what ``AdaptiveStepSizeController._decide`` returns, ``None`` for accept and status."""
    if norm_or_none is None:
        ratio = p["norm"](error_scale(p["atol"], p["rtol"], y0, y1, err))
    else:
        ratio = norm_or_none
    ratio = torch.maximum(ratio, torch.full_like(ratio, p["almost_zero"]))
    factor = p["safety"] * ratio ** p["e1"]
    if p["pid"]:
        factor = factor * prev ** p["e2"] * pprev ** p["e3"]
    dt_next = dt * torch.clamp(factor, min=p["factor_min"], max=p["factor_max"]).to(dt.dtype)
    if p["dt_min"] is not None or p["dt_max"] is not None:
        dt_next = torch.sign(dt_next) * torch.clamp(dt_next.abs(), p["dt_min"], p["dt_max"])
    if not p["pid"]:
        return None, dt_next, ratio, None
    return None, dt_next, ratio, None, torch.where(accept, ratio, prev), torch.where(accept, prev, pprev)


def _direction(t_start, t_end, dtype):
    return torch.where(t_end > t_start, 1.0, -1.0).to(dtype)


def _first_guess(t_start, t_end, d0, d1):
    small = torch.full_like(d0, 1e-6)
    h0 = torch.where((d0 < 1e-5) | (d1 < 1e-5), small, 0.01 * d0 / d1)
    return torch.minimum(h0, (t_end - t_start).abs().to(h0.dtype))


def _probe(t_start, t_end, y0, f0, h0):
    y1 = y0 + (_direction(t_start, t_end, h0.dtype) * h0)[:, None] * f0
    return y1, t_start + _direction(t_start, t_end, t_start.dtype) * h0.to(t_start.dtype)


def initial_step_a(norm: Callable, atol: float, rtol: float, t_start, t_end, y0, f0):
    """reference step_size_controllers.py:459-479: the first guess ``h0`` and the probe point."""
    inv = torch.reciprocal(atol + rtol * y0.abs())
    h0 = _first_guess(t_start, t_end, norm(y0 * inv), norm(f0 * inv))
    return (h0, *_probe(t_start, t_end, y0, f0, h0))


def initial_step_a_norms(t_start, t_end, y0, f0, d0, d1):
    h0 = _first_guess(t_start, t_end, d0, d1)
    return (h0, *_probe(t_start, t_end, y0, f0, h0))


def _finish(guards_zero_step: bool, order: int, t_start, t_end, h0, d1, d2_times_h0):
    d2 = d2_times_h0 / h0
    if guards_zero_step:  # (the integral controller's copy has this line, the PID controller's has not: :481 / :826)
        d2 = torch.where(h0 == 0, torch.full_like(d2, float("inf")), d2)
    m = torch.maximum(d1, d2)
    h1 = torch.where(m <= 1e-15, torch.maximum(torch.full_like(h0, 1e-6), h0 * 1e-3), (0.01 / m) ** (1.0 / order))
    return (_direction(t_start, t_end, h0.dtype) * torch.minimum(100 * h0, h1)).to(t_start.dtype)


def initial_step_b(norm: Callable, guards_zero_step: bool, order: int, atol: float, rtol: float, t_start, t_end, y0, f0, f1, h0):
    """reference step_size_controllers.py:481-490."""
    inv = torch.reciprocal(atol + rtol * y0.abs())
    return _finish(guards_zero_step, order, t_start, t_end, h0, norm(f0 * inv), norm((f1 - f0) * inv))


def initial_step_b_norms(guards_zero_step: bool, order: int, t_start, t_end, h0, d1, d2n):
    return _finish(guards_zero_step, order, t_start, t_end, h0, d1, d2n)


def quartic_from_mid(dt, y0, y1, k_first, k_last, y_mid):
    """reference interpolation.py:152-168: quartic through both ends, their slopes and the mid point."""
    h = dt.to(y0.dtype)[:, None]
    f0, f1 = h * k_first, h * k_last
    return torch.stack((
        y0,
        f0,
        f1.add(f0, alpha=-4).add(y0, alpha=-11).add(y1, alpha=-5).add(y_mid, alpha=16),
        (5 * f0).add(f1, alpha=-3).add(y0, alpha=18).add(y1, alpha=14).add(y_mid, alpha=-32),
        (2 * (f1 - f0)).add(y1 + y0, alpha=-8).add(y_mid, alpha=16),
    ))  # fmt: skip


def quartic_build(mid_weights: Optional[Sequence[float]], theta_weights: Optional[Sequence[Sequence[float]]], dt, y0, y1, *ks):
    """Dense output of a 7-stage pair: through the mid point (reference dopri5.py:53-60) or from the pair's own
    weights of theta^2 .. theta^4 (tsit5.py:123-139)."""
    if mid_weights is not None:
        return quartic_from_mid(dt, y0, y1, ks[0], ks[-1], combine(mid_weights, dt, y0, *ks))
    h = dt.to(y0.dtype)[:, None]
    return torch.stack((y0, h * ks[0], *(h * _weighted_sum(row, ks) for row in theta_weights)))


def cubic_build(dt, y0, y1, k_first, k_last):
    """reference interpolation.py:84-101: the Hermite cubic of a step."""
    h = dt.to(y0.dtype)[:, None]
    gap = y0 - y1
    cube = torch.add(h * (k_first + k_last), gap, alpha=2)
    square = torch.add(h * torch.add(-k_last, k_first, alpha=-2), gap, alpha=-3)
    return torch.stack((y0, h * k_first, square, cube))


def poly_eval(span_is_dt: bool, idx: torch.Tensor, coefficients, t0, t1, t):
    """reference interpolation.py:8-40, 54-60: Horner in ``x = (t - t0) / (t1 - t0)`` on the rows ``idx``."""
    den = t1[idx] if span_is_dt else t1[idx] - t0[idx]
    den = torch.where(den.abs() > 0.0, den, torch.ones_like(den))
    x = ((t - t0[idx]) / den)[:, None].to(coefficients.dtype)
    out = coefficients[-1][idx]
    for p in range(coefficients.shape[0] - 2, -1, -1):
        out = out * x + coefficients[p][idx]
    return out


def loop_begin(t_start, t_end, dt):
    """reference adjoints.py:66-67, 107: the first step kept inside the time range."""
    return torch.clamp(dt, torch.minimum(t_start, t_end) - t_start, torch.maximum(t_end, t_start) - t_start)


def loop_advance(to_update: torch.Tensor, running_next: torch.Tensor, t_start, t_end, t, dt, y, y_new, dt_next):
    """reference adjoints.py:150-152, 247-251 with the iteration's decisions given."""
    t_out = torch.where(to_update, t + dt, t)
    y_out = torch.where(to_update[:, None], y_new, y)
    dt_out = torch.where(running_next, dt_next, dt)
    dt_out = torch.clamp(dt_out, torch.minimum(t_start, t_end) - t_out, torch.maximum(t_end, t_start) - t_out)
    return t_out, dt_out, y_out
