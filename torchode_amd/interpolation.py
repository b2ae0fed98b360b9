"""Local interpolants of a single step (mirror torchode/interpolation.py).

An interpolant answers ``evaluate(t, idx)``: the value of sample ``idx[n]``'s step
polynomial at time ``t[n]``.  The polynomial classes keep their coefficients as one
``[degree+1, B, F]`` device tensor and evaluate with one kernel; any other object with
an ``evaluate`` method can be returned by a user-defined step method instead.
"""
from typing import Sequence, Union

import torch

from . import _lib, differentiable


def _poly_eval_rows(coefficients, t, t0, t1):
    """Row n of the coefficient tensors belongs to time ``t[n]`` on ``[t0[n], t1[n]]``."""
    rows = torch.arange(t.shape[0], device=t.device)
    return _PolynomialInterpolation._make(len(coefficients) - 1, t0, t1, coefficients).evaluate(t, rows)


def poly3eval(d, c, b, a, t, t0, t1):
    """``d + c x + b x^2 + a x^3`` with ``x = (t - t0) / (t1 - t0)``, row by row (reference interpolation.py:8-22)."""
    return _poly_eval_rows((d, c, b, a), t, t0, t1)


def poly4eval(e, d, c, b, a, t, t0, t1):
    """The same with five coefficients, constant term first (reference interpolation.py:25-40)."""
    return _poly_eval_rows((e, d, c, b, a), t, t0, t1)


class LocalInterpolation:
    """Protocol (reference interpolation.py:43-45)."""

    def evaluate(self, t: torch.Tensor, idx: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError()


def _stack(coefficients: Union[torch.Tensor, Sequence[torch.Tensor]]) -> torch.Tensor:
    if isinstance(coefficients, torch.Tensor):
        return coefficients.contiguous()
    return torch.stack(list(coefficients)).contiguous()


class _PolynomialInterpolation(LocalInterpolation):
    """Polynomial on [t0, t1] in x = (t - t0) / (t1 - t0); ``coefficients[i]`` belongs to x**i."""

    degree = -1
    span_is_dt = 0  # 1: the second time operand is the step size and divides as it stands

    def __init__(self, t0: torch.Tensor, t1: torch.Tensor, coefficients):
        self.t0 = t0
        self.t1 = t1
        self._coeff = _stack(coefficients)
        assert self._coeff.ndim == 3 and self._coeff.shape[0] == self.degree + 1
        self.coefficients = tuple(self._coeff.unbind(0))

    @staticmethod
    def _make(degree: int, t0, t1, coefficients) -> "_PolynomialInterpolation":
        cls = type("_Polynomial", (_PolynomialInterpolation,), {"degree": degree})
        return cls(t0, t1, coefficients)

    def _span(self) -> torch.Tensor:
        return self.t1

    def _code(self, *times) -> int:
        c = self._coeff
        _lib.require_device(c, self.t0, self.t1, *times)
        assert all(t.dtype == self.t0.dtype for t in (self.t1, *times)), "time tensors of different dtypes"
        return _lib.dtype_code(c.dtype, self.t0.dtype)

    def tracked(self, *times) -> bool:
        """True if values of this polynomial have to carry a graph (then ``evaluate`` is the way to them)."""
        return differentiable.tracked(self._coeff, self.t0, self._span(), *times)

    def evaluate(self, t: torch.Tensor, idx: torch.Tensor) -> torch.Tensor:
        """reference interpolation.py:103-106, 172-175"""
        code = self._code(t)
        idx = idx.to(torch.long).contiguous()

        def kernel():
            c = self._coeff
            _, B, F = c.shape
            t_, t0, t1 = t.contiguous(), self.t0.contiguous(), self._span().contiguous()
            out = c.new_empty((t_.shape[0], F))
            rc = _lib.load().tode_poly_eval(
                code, self.degree, self.span_is_dt, B, F, t_.shape[0], _lib.ptr(c), _lib.ptr(t0), _lib.ptr(t1), _lib.ptr(t_),
                _lib.ptr(idx), _lib.ptr(out), _lib.stream_of(c),
            )  # fmt: skip
            _lib.check(rc, "tode_poly_eval")
            return out

        formula = lambda c, t0, t1, t_: differentiable.poly_eval(bool(self.span_is_dt), idx, c, t0, t1, t_)
        return differentiable.through(kernel, formula, self._coeff, self.t0, self._span(), t)

    def evaluate_masked(self, t_eval: torch.Tensor, mask: torch.Tensor, ys: torch.Tensor) -> None:
        """``ys[b, e] = p_b(t_eval[b, e])`` wherever ``mask[b, e]`` is set (one byte per entry);
        the index list of reference adjoints.py:227-233 is never materialised."""
        code = self._code(t_eval)
        c = self._coeff
        _, B, F = c.shape
        assert t_eval.is_contiguous() and mask.is_contiguous() and ys.is_contiguous() and mask.element_size() == 1
        t0, t1 = self.t0.contiguous(), self._span().contiguous()
        rc = _lib.load().tode_poly_eval_masked(
            code, self.degree, self.span_is_dt, B, F, t_eval.shape[1], _lib.ptr(c), _lib.ptr(t0), _lib.ptr(t1),
            _lib.ptr(t_eval), _lib.ptr(mask), _lib.ptr(ys), _lib.stream_of(c),
        )  # fmt: skip
        _lib.check(rc, "tode_poly_eval_masked")

    def __repr__(self):
        return f"{type(self).__name__}(t0={self.t0}, t1={self.t1}, coefficients={self.coefficients})"


def _build_args(dt, y0, y1, *more):
    """Contiguous operands and the dtype code (dt in the time dtype, the rest in the data dtype)."""
    _lib.require_device(dt, y0, y1, *more)
    assert all(x.dtype == y0.dtype for x in (y1, *more)), "data tensors of different dtypes"
    return [_lib.dtype_code(y0.dtype, dt.dtype)] + [x.contiguous() for x in (dt, y0, y1, *more)]


class LinearInterpolation(_PolynomialInterpolation):
    """y0 + (y1 - y0) x with x = (t - t0) / dt: the step size itself divides, not (t0 + dt) - t0, which can differ
    from it in the last bit (reference interpolation.py:48-62)."""

    degree = 1
    span_is_dt = 1

    def __init__(self, t0: torch.Tensor, dt: torch.Tensor, y0: torch.Tensor, y1: torch.Tensor):
        self.dt = dt
        super().__init__(t0, t0 + dt, (y0, y1 - y0))
        self.y0 = y0
        self.dy = self.coefficients[1]

    def _span(self) -> torch.Tensor:
        return self.dt


class ThirdOrderPolynomialInterpolation(_PolynomialInterpolation):
    """reference interpolation.py:65-118"""

    degree = 3

    @staticmethod
    def from_k(t0, dt, y0, y1, k):
        """Hermite cubic from the first and last stage derivative (reference interpolation.py:84-106)."""
        k_first, k_last = k[0], k[-1]

        def kernel():
            code, dt_, y0_, y1_, kf, kl = _build_args(dt, y0, y1, k_first, k_last)
            B, F = y0_.shape
            coeff = y0_.new_empty((4, B, F))
            rc = _lib.load().tode_cubic_build(
                code, B, F, _lib.ptr(dt_), _lib.ptr(y0_), _lib.ptr(y1_), _lib.ptr(kf), _lib.ptr(kl),
                _lib.ptr(coeff), _lib.stream_of(y0_),
            )  # fmt: skip
            _lib.check(rc, "tode_cubic_build")
            return coeff

        coeff = differentiable.through(kernel, differentiable.cubic_build, dt, y0, y1, k_first, k_last)
        return ThirdOrderPolynomialInterpolation(t0, t0 + dt, coeff)


class FourthOrderPolynomialInterpolation(_PolynomialInterpolation):
    """reference interpolation.py:121-181"""

    degree = 4

    @staticmethod
    def from_k(t0, dt, y0, y1, k, b_mid):
        """Quartic through both end points, their derivatives and the mid-point value
        ``y0 + dt * sum_s b_mid[s] k[s]`` (reference interpolation.py:138-170)."""
        w = [float(x) for x in (b_mid.tolist() if isinstance(b_mid, torch.Tensor) else b_mid)]
        assert len(w) == k.shape[0] <= _lib.MAX_STAGES

        def mid_kernel():
            code, dt_, y0_, y1_, k_ = _build_args(dt, y0, y1, k)
            S, B, F = k_.shape
            y_mid = torch.empty_like(y0_)
            rc = _lib.load().tode_erk_combine(code, B, F, S, (_lib.C.c_double * S)(*w), _lib.ptr(dt_), _lib.ptr(k_), _lib.ptr(y0_), _lib.ptr(y_mid), _lib.stream_of(y0_))
            _lib.check(rc, "tode_erk_combine")
            return y_mid

        y_mid = differentiable.through(mid_kernel, lambda dt_, y0_, k_: differentiable.combine(w, dt_, y0_, *k_.unbind(0)), dt, y0, k)
        k_first, k_last = k[0], k[-1]

        def kernel():
            code, dt_, y0_, y1_, kf, kl, mid = _build_args(dt, y0, y1, k_first, k_last, y_mid)
            B, F = y0_.shape
            coeff = y0_.new_empty((5, B, F))
            rc = _lib.load().tode_quartic_from_mid(
                code, B, F, _lib.ptr(dt_), _lib.ptr(y0_), _lib.ptr(y1_), _lib.ptr(kf), _lib.ptr(kl), _lib.ptr(mid),
                _lib.ptr(coeff), _lib.stream_of(y0_),
            )  # fmt: skip
            _lib.check(rc, "tode_quartic_from_mid")
            return coeff

        coeff = differentiable.through(kernel, differentiable.quartic_from_mid, dt, y0, y1, k_first, k_last, y_mid)
        return FourthOrderPolynomialInterpolation(t0, t0 + dt, coeff)

    @staticmethod
    def from_erk_step(method_id: int, t0, dt, y0, y1, k):
        """Dense output of a Dopri5 / Tsit5 step with the pair's own weights, one kernel
        (reference tsit5.py:123-139, dopri5.py:53-60)."""
        assert k.shape[0] == 7

        def kernel():
            code, dt_, y0_, y1_, k_ = _build_args(dt, y0, y1, k)
            S, B, F = k_.shape
            coeff = y0_.new_empty((5, B, F))
            rc = _lib.load().tode_quartic_build(
                code, method_id, B, F, _lib.ptr(dt_), _lib.ptr(y0_), _lib.ptr(y1_), _lib.ptr(k_), _lib.ptr(coeff),
                _lib.stream_of(y0_),
            )  # fmt: skip
            _lib.check(rc, "tode_quartic_build")
            return coeff

        def formula(dt_, y0_, y1_, k_):
            from .single_step_methods.runge_kutta import library_tableau

            rows = library_tableau(method_id).b_other.tolist()  # Dopri5: the mid-point weights; Tsit5: theta^2 .. theta^4
            mid, theta = (rows[0], None) if len(rows) == 1 else (None, rows)
            return differentiable.quartic_build(mid, theta, dt_, y0_, y1_, *k_.unbind(0))

        coeff = differentiable.through(kernel, formula, dt, y0, y1, k)
        return FourthOrderPolynomialInterpolation(t0, t0 + dt, coeff)
