"""Step size controllers (mirror torchode/step_size_controllers.py).

The classes keep the reference's constructor signatures and protocol methods
(``init``, ``adapt_step_size``, ``merge_states`` ...).  Their arithmetic runs in HIP
kernels: inside the whole-solve kernel when ``AutoDiffAdjoint`` recognises the whole
configuration, and one kernel per protocol call otherwise.  A user-defined controller
subclasses ``StepSizeController``.
"""
from functools import partial
from math import sqrt
from typing import Any, Callable, Dict, NamedTuple, Optional, Tuple

import torch
import torch.nn as nn

from . import _lib, differentiable
from .problems import InitialValueProblem
from .terms import ODETerm


def rms_norm(y: torch.Tensor) -> torch.Tensor:
    """Root mean square norm over the feature dimension (Hairer, Norsett & Wanner I, eq. II.4.11;
    reference step_size_controllers.py:170-181).  Passing this function as ``norm`` (the default)
    selects the fused kernels, which compute the same quantity on the device."""
    return torch.linalg.vector_norm(y / sqrt(y.shape[1]), ord=2, dim=1)


def max_norm(y: torch.Tensor) -> torch.Tensor:
    """Maximum norm over the feature dimension (reference step_size_controllers.py:184-186)."""
    return torch.linalg.vector_norm(y, dim=1, ord=torch.inf)


class StepSizeController(nn.Module):
    """Protocol (reference step_size_controllers.py:16-113)."""

    def init(self, term: Optional[ODETerm], problem: InitialValueProblem, method_order: int, dt0: Optional[torch.Tensor], *, stats: Dict[str, Any], args: Any):
        """Returns ``(dt0, controller state, f(t_start, y0) or None)``; a step size suggested by the user wins."""
        raise NotImplementedError()

    def adapt_step_size(self, t0, dt, y0, step_result, state, stats: Dict[str, Any]):
        """Returns ``(accept [B] bool, next dt [B], next state, status int64 [B] or None)``."""
        raise NotImplementedError()

    def merge_states(self, running: torch.Tensor, current, previous):
        """State that is ``current`` for samples still running and ``previous`` for finished ones."""
        raise NotImplementedError()


class FixedStepState(NamedTuple):
    accept_all: torch.Tensor
    dt0: torch.Tensor


class FixedStepController(StepSizeController):
    """Accepts every step and keeps the step size (reference step_size_controllers.py:116-167)."""

    fusable = True  # the per-step kernels know this controller (it has no whole-solve kernel)

    def c_struct(self, limits=None) -> "_lib.Controller":
        """``struct tode_controller`` of kind TODE_CTRL_FIXED; no other field is looked at."""
        return _lib.Controller(_lib.CTRL_FIXED, False, False, 0, 0.0, 0.0, 0.0, 1.0, 0.0, 0.9, 0.2, 10.0, 0.0, 0.0)

    def init(self, term, problem, method_order, dt0, *, stats, args):
        assert dt0 is not None, "Fixed step size solving requires you to configure dt0"
        accept_all = torch.ones(problem.batch_size, device=problem.device, dtype=torch.bool)
        return dt0, FixedStepState(accept_all=accept_all, dt0=dt0), None

    def adapt_step_size(self, t0, dt, y0, step_result, state: FixedStepState, stats):
        return state.accept_all, state.dt0, state, None

    def merge_states(self, running, current: FixedStepState, previous: FixedStepState):
        return current


def _almost_zero(dtype, device):
    # lower bound of the error ratio (reference step_size_controllers.py:243-249)
    return torch.tensor(1e-5 if dtype == torch.float16 else 1e-38, dtype=dtype, device=device)


def _limit(x):
    return None if x is None else float(x)


class IntegralState:
    """reference step_size_controllers.py:215-257"""

    def __init__(self, method_order: int, almost_zero: torch.Tensor, dt_min=None, dt_max=None):
        self.method_order = method_order
        self.almost_zero = almost_zero
        self.dt_min = dt_min
        self.dt_max = dt_max

    def update_error_ratios(self, prev_error_ratio, prev_prev_error_ratio):
        return self

    def __repr__(self):
        return f"IState(method_order={self.method_order}, almost_zero={self.almost_zero}, dt_min={self.dt_min}, dt_max={self.dt_max})"

    @staticmethod
    def default(*, method_order: int, batch_size: int, dtype, device, dt_min, dt_max):
        return IntegralState(method_order, _almost_zero(dtype, device), dt_min, dt_max)


class PIDState:
    """reference step_size_controllers.py:493-551: the error ratios of the last two accepted steps"""

    def __init__(self, method_order: int, prev_error_ratio, prev_prev_error_ratio, almost_zero, dt_min=None, dt_max=None):
        self.method_order = method_order
        self.prev_error_ratio = prev_error_ratio
        self.prev_prev_error_ratio = prev_prev_error_ratio
        self.almost_zero = almost_zero
        self.dt_min = dt_min
        self.dt_max = dt_max

    def update_error_ratios(self, prev_error_ratio, prev_prev_error_ratio):
        return PIDState(self.method_order, prev_error_ratio, prev_prev_error_ratio, self.almost_zero, self.dt_min, self.dt_max)

    def __repr__(self):
        return (
            f"PIDState(method_order={self.method_order}, prev_error_ratio={self.prev_error_ratio}, "
            f"prev_prev_error_ratio={self.prev_prev_error_ratio}, almost_zero={self.almost_zero}, "
            f"dt_min={self.dt_min}, dt_max={self.dt_max})"
        )

    @staticmethod
    def default(*, method_order: int, batch_size: int, dtype, device, dt_min, dt_max):
        ones = torch.ones(batch_size, dtype=dtype, device=device)
        return PIDState(method_order, ones, ones, _almost_zero(dtype, device), dt_min, dt_max)


class AdaptiveStepSizeController(StepSizeController):
    """Error-ratio based control shared by the integral and the PID controller
    (reference step_size_controllers.py:189-213, 333-490, 678-835)."""

    _kind = -1

    def __init__(self, atol, rtol, pcoeff, icoeff, dcoeff, term, norm, dt_min, dt_max, safety, factor_min, factor_max):
        super().__init__()
        # float32 buffers, as in the reference: the tolerances take effect float32-rounded
        # even in a float64 solve
        self.register_buffer("atol", torch.tensor(atol))
        self.register_buffer("rtol", torch.tensor(rtol))
        self.term = term
        self.norm = norm
        self.dt_min = dt_min
        self.dt_max = dt_max
        self.pcoeff = pcoeff
        self.icoeff = icoeff
        self.dcoeff = dcoeff
        self.safety = safety
        self.factor_min = factor_min
        self.factor_max = factor_max
        self._atol_f = float(torch.tensor(atol))
        self._rtol_f = float(torch.tensor(rtol))

    # ------------------------------------------------------------------ #
    @property
    def fusable(self) -> bool:
        """True when the whole-solve kernels implement this controller exactly (RMS norm)."""
        return self.norm is rms_norm

    def _norm_id(self) -> Optional[int]:
        return {rms_norm: _lib.NORM_RMS, max_norm: _lib.NORM_MAX}.get(self.norm)

    def c_struct(self, limits=None) -> "_lib.Controller":
        """Parameters in the layout of ``struct tode_controller``.  ``limits`` is a
        ``(dt_min, dt_max)`` pair of floats or ``None``s; by default the constructor's."""
        dt_min, dt_max = (self.dt_min, self.dt_max) if limits is None else limits
        return _lib.Controller(
            self._kind, dt_min is not None, dt_max is not None, 0, self._atol_f, self._rtol_f,
            float(self.pcoeff), float(self.icoeff), float(self.dcoeff), float(self.safety),
            float(self.factor_min), float(self.factor_max), float(dt_min or 0.0), float(dt_max or 0.0),
        )  # fmt: skip

    def control_values(self):
        """``(kind, values)``: the same parameters as plain Python numbers, in the order of ``struct tode_controller``
        with NaN for a step size limit that is not set, as ``torch.ops.torchode_amd.solve_builtin`` takes them."""
        nan = float("nan")
        return self._kind, [
            self._atol_f, self._rtol_f, float(self.pcoeff), float(self.icoeff), float(self.dcoeff), float(self.safety), float(self.factor_min),
            float(self.factor_max), nan if self.dt_min is None else float(self.dt_min), nan if self.dt_max is None else float(self.dt_max),
        ]  # fmt: skip

    # ------------------------------------------------------------------ #
    def initial_state(self, method_order: int, problem: InitialValueProblem, dt_min, dt_max):
        raise NotImplementedError()

    def update_state(self, state, y0, dt, error_ratio, accept):
        raise NotImplementedError()

    def _decide(self, state, dt, *, norm=None, y0=None, y1=None, err=None, limits=True, data_dtype=None):
        """Runs the decision kernel: fused with the error norm when ``norm`` is None, from a
        precomputed norm otherwise.  Returns (accept, dt_next, ratio, status, prev, prev_prev)."""
        _lib.require_device(dt, norm, y0, y1, err)
        data_dtype = data_dtype if y0 is None else y0.dtype
        code = _lib.dtype_code(data_dtype, dt.dtype)
        B = dt.shape[0]
        pid = self._kind == _lib.CTRL_PID
        prev = state.prev_error_ratio.to(data_dtype) if pid else None
        pprev = state.prev_prev_error_ratio.to(data_dtype) if pid else None
        # the limits in force are the state's (reference step_size_controllers.py:406-408)
        c = self.c_struct((_limit(state.dt_min), _limit(state.dt_max)) if limits else (None, None))
        order = int(state.method_order)
        decided = {}

        def kernel():
            dt_ = dt.contiguous()
            accept = torch.empty(B, dtype=torch.bool, device=dt.device)
            dt_next, ratio = torch.empty_like(dt_), torch.empty(B, dtype=data_dtype, device=dt.device)
            status = torch.empty(B, dtype=torch.long, device=dt.device)
            prev_, pprev_ = (prev.contiguous(), pprev.contiguous()) if pid else (None, None)
            prev_o = torch.empty_like(ratio) if pid else None
            pprev_o = torch.empty_like(ratio) if pid else None
            lib, stream = _lib.load(), _lib.stream_of(dt)
            tail = (_lib.ptr(prev_), _lib.ptr(pprev_), _lib.ptr(accept), _lib.ptr(dt_next), _lib.ptr(ratio), _lib.ptr(status),
                    _lib.ptr(prev_o), _lib.ptr(pprev_o), stream)  # fmt: skip
            if norm is None:
                a, b, e = (x.contiguous() for x in (y0, y1, err))
                assert b.dtype == a.dtype == e.dtype and a.shape == b.shape == e.shape
                rc = lib.tode_adapt_step(code, _lib.C.byref(c), order, self._norm_id(), B, a.shape[1], _lib.ptr(dt_), _lib.ptr(a), _lib.ptr(b), _lib.ptr(e), *tail)
                _lib.check(rc, "tode_adapt_step")
            else:
                n = norm.to(data_dtype).contiguous()
                rc = lib.tode_control(code, _lib.C.byref(c), order, B, _lib.ptr(n), _lib.ptr(dt_), *tail)
                _lib.check(rc, "tode_control")
            decided["accept"] = accept
            return (accept, dt_next, ratio, status, prev_o, pprev_o) if pid else (accept, dt_next, ratio, status)

        def formula(dt_, norm_, y0_, y1_, err_, prev_, pprev_):
            k_i, k_p, k_d = float(self.icoeff) / order, float(self.pcoeff) / order, float(self.dcoeff) / order
            p = dict(
                atol=self._atol_f, rtol=self._rtol_f, norm={_lib.NORM_RMS: differentiable.rms, _lib.NORM_MAX: differentiable.maximum_norm}.get(self._norm_id()),
                almost_zero=float(state.almost_zero), safety=float(self.safety), pid=pid, factor_min=float(self.factor_min), factor_max=float(self.factor_max),
                e1=-(k_i + k_p + k_d) if pid else -1.0 / order, e2=k_p + 2 * k_d, e3=-k_d,
                dt_min=_limit(state.dt_min) if limits else None, dt_max=_limit(state.dt_max) if limits else None,
            )  # fmt: skip
            return differentiable.decide(p, decided["accept"], dt_, None if norm_ is None else norm_.to(data_dtype), y0_, y1_, err_, prev_, pprev_)

        out = differentiable.through(kernel, formula, dt, norm, y0, y1, err, prev, pprev)
        return out if pid else (*out, None, None)

    def dt_factor(self, state, error_ratio: torch.Tensor) -> torch.Tensor:
        """Growth factor of the step size for a given error ratio, clipped to
        ``[factor_min, factor_max]`` (reference step_size_controllers.py:289-294, 598-621)."""
        ones = torch.ones_like(error_ratio)
        return self._decide(state, ones, norm=error_ratio, limits=False, data_dtype=error_ratio.dtype)[1]

    # ------------------------------------------------------------------ #
    def init(self, term, problem: InitialValueProblem, method_order: int, dt0, *, stats, args):
        """reference step_size_controllers.py:333-368, 678-713"""
        if dt0 is None:
            dt0, f0 = self._select_initial_step(term, problem, method_order, stats, args)
        else:
            f0 = None
        dt_min, dt_max = self.dt_min, self.dt_max
        if dt_min is not None:
            dt_min = torch.tensor(dt_min, dtype=problem.time_dtype, device=problem.device)
        if dt_max is not None:
            dt_max = torch.tensor(dt_max, dtype=problem.time_dtype, device=problem.device)
        return dt0, self.initial_state(method_order, problem, dt_min, dt_max), f0

    def adapt_step_size(self, t0, dt, y0, step_result, state, stats):
        """reference step_size_controllers.py:370-429, 715-774"""
        y1, error_estimate = step_result.y, step_result.error_estimate
        if error_estimate is None:
            # no error estimate: accept and keep the step size
            return torch.ones_like(dt, dtype=torch.bool), dt, self.update_state(state, y0, dt, None, None), None
        if self._norm_id() is not None:
            accept, dt_next, ratio, status, prev, pprev = self._decide(state, dt, y0=y0, y1=y1, err=error_estimate)
        else:
            # user-defined norm: scale on the device, call the norm, decide on the device
            _lib.require_device(y0, y1, error_estimate)
            if y0.dtype not in _lib.DTYPES or not (y0.dtype == y1.dtype == error_estimate.dtype):
                raise NotImplementedError("the step size controllers need float32 or float64 data of one dtype")

            def scale_kernel():
                a, b, e = y0.contiguous(), y1.contiguous(), error_estimate.contiguous()
                scaled = torch.empty_like(a)
                rc = _lib.load().tode_error_scale(
                    _lib.DTYPES[a.dtype], a.shape[0], a.shape[1], self._atol_f, self._rtol_f, _lib.ptr(a), _lib.ptr(b), _lib.ptr(e),
                    _lib.ptr(scaled), _lib.stream_of(a),
                )  # fmt: skip
                _lib.check(rc, "tode_error_scale")
                return scaled

            scaled = differentiable.through(scale_kernel, partial(differentiable.error_scale, self._atol_f, self._rtol_f), y0, y1, error_estimate)
            accept, dt_next, ratio, status, prev, pprev = self._decide(state, dt, norm=self.norm(scaled), data_dtype=y0.dtype)
        if self._kind == _lib.CTRL_PID and type(self).update_state is PIDController.update_state:
            state = state.update_error_ratios(prev, pprev)  # the decision kernel has already shifted the history
        else:
            state = self.update_state(state, y0, dt, ratio, accept)
        return accept, dt_next, state, status

    def _select_initial_step(self, term, problem: InitialValueProblem, method_order: int, stats, args):
        """Hairer, Norsett & Wanner I, Sec. II.4, with the tolerances applied to the norms
        (reference step_size_controllers.py:431-490, 776-835).  Two kernels around the two
        evaluations of ``f``."""
        term_ = term if term is not None else self.term
        assert term_ is not None
        norm = self._norm_id()
        y0, t0, t1 = problem.y0.contiguous(), problem.t_start.contiguous(), problem.t_end.contiguous()
        _lib.require_device(y0, t0, t1)
        B, F = y0.shape
        lib, code, stream = _lib.load(), _lib.dtype_code(y0.dtype, t0.dtype), _lib.stream_of(y0)
        atol, rtol, order = self._atol_f, self._rtol_f, int(method_order)
        guards = self._kind == _lib.CTRL_INTEGRAL  # (only the integral controller's copy treats a zero first guess, :481 / :826)
        f0 = term_.vf(t0, y0, stats, args).to(y0.dtype).contiguous()
        if norm is None:
            # user-defined norm: its arguments are scaled on the device, it is called three times
            def scaled_norm(v):
                def kernel():
                    out = torch.empty_like(y0)
                    rc = lib.tode_tolerance_scale(code, B, F, atol, rtol, _lib.ptr(y0), _lib.ptr(v), _lib.ptr(out), stream)
                    _lib.check(rc, "tode_tolerance_scale")
                    return out

                return self.norm(differentiable.through(kernel, partial(differentiable.tolerance_scale, atol, rtol), y0, v)).to(y0.dtype).contiguous()

            d0, d1 = scaled_norm(y0), scaled_norm(f0)

            def probe_kernel():
                h0, y1, tn = y0.new_empty(B), torch.empty_like(y0), torch.empty_like(t0)
                rc = lib.tode_initial_step_a_norms(
                    code, B, F, _lib.ptr(t0), _lib.ptr(t1), _lib.ptr(y0), _lib.ptr(f0), _lib.ptr(d0), _lib.ptr(d1), _lib.ptr(h0),
                    _lib.ptr(y1), _lib.ptr(tn), stream,
                )  # fmt: skip
                _lib.check(rc, "tode_initial_step_a_norms")
                return h0, y1, tn

            h0, y1, tn = differentiable.through(probe_kernel, differentiable.initial_step_a_norms, t0, t1, y0, f0, d0, d1)
            f1 = term_.vf(tn, y1, stats, args).to(y0.dtype).contiguous()
            d2n = scaled_norm(f1 - f0)

            def finish_kernel():
                dt0 = torch.empty_like(t0)
                rc = lib.tode_initial_step_b_norms(
                    code, self._kind, order, B, _lib.ptr(t0), _lib.ptr(t1), _lib.ptr(h0), _lib.ptr(d1), _lib.ptr(d2n),
                    _lib.ptr(dt0), stream,
                )  # fmt: skip
                _lib.check(rc, "tode_initial_step_b_norms")
                return dt0

            return differentiable.through(finish_kernel, partial(differentiable.initial_step_b_norms, guards, order), t0, t1, h0, d1, d2n), f0
        norm_formula = {_lib.NORM_RMS: differentiable.rms, _lib.NORM_MAX: differentiable.maximum_norm}[norm]

        def probe_kernel():
            h0, y1, tn = y0.new_empty(B), torch.empty_like(y0), torch.empty_like(t0)
            rc = lib.tode_initial_step_a(
                code, norm, B, F, atol, rtol, _lib.ptr(t0), _lib.ptr(t1), _lib.ptr(y0), _lib.ptr(f0),
                _lib.ptr(h0), _lib.ptr(y1), _lib.ptr(tn), stream,
            )  # fmt: skip
            _lib.check(rc, "tode_initial_step_a")
            return h0, y1, tn

        h0, y1, tn = differentiable.through(probe_kernel, partial(differentiable.initial_step_a, norm_formula, atol, rtol), t0, t1, y0, f0)
        f1 = term_.vf(tn, y1, stats, args).to(y0.dtype).contiguous()

        def finish_kernel():
            dt0 = torch.empty_like(t0)
            rc = lib.tode_initial_step_b(
                code, self._kind, norm, order, B, F, atol, rtol, _lib.ptr(t0), _lib.ptr(t1),
                _lib.ptr(y0), _lib.ptr(f0), _lib.ptr(f1), _lib.ptr(h0), _lib.ptr(dt0), stream,
            )  # fmt: skip
            _lib.check(rc, "tode_initial_step_b")
            return dt0

        dt0 = differentiable.through(finish_kernel, partial(differentiable.initial_step_b, norm_formula, guards, order, atol, rtol), t0, t1, y0, f0, f1, h0)
        return dt0, f0


# name kept for the dispatch in adjoints.py
_AdaptiveController = AdaptiveStepSizeController


class IntegralController(AdaptiveStepSizeController):
    """Scales the step by ``safety * ratio**(-1/order)`` clipped to ``[factor_min, factor_max]``
    (reference step_size_controllers.py:260-294)."""

    _kind = _lib.CTRL_INTEGRAL

    def __init__(
        self,
        atol: float,
        rtol: float,
        *,
        term: Optional[ODETerm] = None,
        norm: Callable = rms_norm,
        dt_min: Optional[float] = None,
        dt_max: Optional[float] = None,
        safety: float = 0.9,
        factor_min: float = 0.2,
        factor_max: float = 10.0,
    ):
        super().__init__(atol, rtol, 0.0, 1.0, 0.0, term, norm, dt_min, dt_max, safety, factor_min, factor_max)

    def initial_state(self, method_order: int, problem: InitialValueProblem, dt_min, dt_max) -> IntegralState:
        return IntegralState.default(
            method_order=method_order, batch_size=problem.batch_size, dtype=problem.data_dtype, device=problem.device,
            dt_min=dt_min, dt_max=dt_max,
        )  # fmt: skip

    def merge_states(self, running, current: IntegralState, previous: IntegralState) -> IntegralState:
        return current

    def update_state(self, state: IntegralState, y0, dt, error_ratio, accept) -> IntegralState:
        return state


class PIDController(AdaptiveStepSizeController):
    """PID step size control after Soederlind (2003), eq. (34), with the coefficients divided by
    the method order (reference step_size_controllers.py:554-620)."""

    _kind = _lib.CTRL_PID

    def __init__(
        self,
        atol: float,
        rtol: float,
        pcoeff: float,
        icoeff: float,
        dcoeff: float,
        *,
        term: Optional[ODETerm] = None,
        norm: Callable = rms_norm,
        dt_min: Optional[float] = None,
        dt_max: Optional[float] = None,
        safety: float = 0.9,
        factor_min: float = 0.2,
        factor_max: float = 10.0,
    ):
        super().__init__(atol, rtol, pcoeff, icoeff, dcoeff, term, norm, dt_min, dt_max, safety, factor_min, factor_max)

    def initial_state(self, method_order: int, problem: InitialValueProblem, dt_min, dt_max) -> PIDState:
        return PIDState.default(
            method_order=method_order, batch_size=problem.batch_size, dtype=problem.data_dtype, device=problem.device,
            dt_min=dt_min, dt_max=dt_max,
        )  # fmt: skip

    def merge_states(self, running, current: PIDState, previous: PIDState) -> PIDState:
        """reference step_size_controllers.py:628-638"""
        pairs = ((current.prev_error_ratio, previous.prev_error_ratio), (current.prev_prev_error_ratio, previous.prev_prev_error_ratio))
        return current.update_error_ratios(*(_select(running, cur, prev) for cur, prev in pairs))

    def update_state(self, state: PIDState, y0, dt, error_ratio, accept) -> PIDState:
        """reference step_size_controllers.py:640-671"""
        if error_ratio is None:
            return state.update_error_ratios(prev_error_ratio=y0.new_ones(dt.shape), prev_prev_error_ratio=state.prev_error_ratio)
        assert accept is not None
        pairs = ((error_ratio, state.prev_error_ratio), (state.prev_error_ratio, state.prev_prev_error_ratio))
        return state.update_error_ratios(*(_select(accept, cur, prev) for cur, prev in pairs))


def _select(mask: torch.Tensor, current: torch.Tensor, previous: torch.Tensor) -> torch.Tensor:
    """``current`` where ``mask`` (one byte per sample), ``previous`` elsewhere."""
    _lib.require_device(current, previous, mask)
    assert mask.element_size() == 1 and current.dtype == previous.dtype and current.dtype in _lib.DTYPES

    def kernel():
        cur, prev, m = current.contiguous(), previous.contiguous(), mask.contiguous()
        out = torch.empty_like(cur)
        rc = _lib.load().tode_select_rows(_lib.DTYPES[cur.dtype], cur.shape[0], 1, _lib.ptr(m), _lib.ptr(cur), _lib.ptr(prev), _lib.ptr(out), _lib.stream_of(cur))
        _lib.check(rc, "tode_select_rows")
        return out

    return differentiable.through(kernel, lambda cur, prev: differentiable.select_rows(mask, cur, prev), current, previous)
