"""Explicit Runge-Kutta methods over a Butcher tableau (mirror torchode/single_step_methods/runge_kutta.py).

The stage inputs, the weighted stage sums and the FSAL merge run as HIP kernels;
the right-hand side is the caller's torch callable, evaluated between them.
"""
from functools import partial
from typing import Any, Dict, List, NamedTuple, Optional

import torch

from .. import _lib, differentiable
from ..problems import InitialValueProblem
from ..terms import ODETerm
from .base import SingleStepMethod, StepResult


# shapes of a tableau's parts, for annotations: c [stages], a [stages, stages], b and b_err [stages], b_other [n, stages]
# (reference runge_kutta.py:15-28: nodes, nodes x weights, weights, rows x weights)
CoefficientVector = RungeKuttaMatrix = WeightVector = WeightMatrix = torch.Tensor


class ButcherTableau:
    """Coefficients as float64 CPU tensors: nodes ``c``, matrix ``a`` (square, strictly lower
    triangular for explicit methods), weights ``b``, error weights ``b_err`` and optional extra
    weight rows ``b_other`` (reference runge_kutta.py:31-166)."""

    def __init__(self, c, a, b, b_err, b_other=None, fsal: Optional[bool] = None, ssal: Optional[bool] = None):
        self.c, self.a, self.b, self.b_err, self.b_other = c, a, b, b_err, b_other
        self.fsal = self.is_fsal() if fsal is None else fsal
        self.ssal = self.is_ssal() if ssal is None else ssal
        self._host = None

    @staticmethod
    def from_lists(
        *, c: List[float], a: List[List[float]], b: List[float], b_err: Optional[List[float]] = None,
        b_low_order: Optional[List[float]] = None, b_other: Optional[List[List[float]]] = None,
    ):  # fmt: skip
        assert b_err is not None or b_low_order is not None, (
            "You have to provide either the weights for the error approximation"
            " or the weights of an embedded lower-order method"
        )
        n = len(c)
        assert n == len(b) and len(a) == n
        a_full = [list(row) + [0.0] * (n - len(row)) for row in a]
        b_t = torch.tensor(b, dtype=torch.float64)
        if b_err is None:
            assert len(b_low_order) == n
            b_err_t = b_t - torch.tensor(b_low_order, dtype=torch.float64)
        else:
            b_err_t = torch.tensor(b_err, dtype=torch.float64)
        b_other_t = None
        if b_other is not None:
            b_other_t = torch.tensor(b_other, dtype=torch.float64)
            assert b_other_t.ndim == 2 and b_other_t.shape[1] == n
        return ButcherTableau(torch.tensor(c, dtype=torch.float64), torch.tensor(a_full, dtype=torch.float64), b_t, b_err_t, b_other_t)

    def to(self, device, time_dtype, data_dtype) -> "ButcherTableau":
        b_other = None if self.b_other is None else self.b_other.to(device, data_dtype)
        out = ButcherTableau(
            self.c.to(device, time_dtype), self.a.to(device, data_dtype), self.b.to(device, data_dtype),
            self.b_err.to(device, data_dtype), b_other, fsal=self.fsal, ssal=self.ssal,
        )  # fmt: skip
        out._host = self.host()
        return out

    def host(self) -> "_HostTableau":
        """Coefficients as Python floats / ctypes arrays for the kernels (made once)."""
        if self._host is None:
            self._host = _HostTableau(self)
        return self._host

    @property
    def n_stages(self):
        return self.c.shape[0]

    def _lower_triangular(self):
        return (torch.triu(self.a, diagonal=1) == 0.0).all().item()

    def is_fsal(self):
        """``f(t0, y0)`` of a step equals the last stage derivative of the previous one."""
        return bool(
            self._lower_triangular() and (self.b == self.a[-1]).all().item() and (self.c[0] == 0.0).item()
            and (self.c[-1] == 1.0).item() and (self.a[0, 0] == 0.0).item()
        )  # fmt: skip

    def is_ssal(self):
        """The solution equals the last stage input."""
        return bool(
            self._lower_triangular() and (self.b == self.a[-1]).all().item() and (self.c[-1] == 1.0).item()
            and (self.a[-1, -1] == 0.0).item()
        )  # fmt: skip


class _HostTableau:
    def __init__(self, tab: ButcherTableau):
        D = _lib.C.c_double
        self.n_stages = int(tab.c.shape[0])
        assert self.n_stages <= _lib.MAX_STAGES, f"at most {_lib.MAX_STAGES} stages"
        assert tab._lower_triangular() and all(tab.a[i, i] == 0 for i in range(self.n_stages)), "explicit tableaux only"
        c64, a64 = tab.c.double().cpu(), tab.a.double().cpu()
        self.c = [float(x) for x in c64]
        self.a_rows = [(D * max(i, 1))(*[float(x) for x in a64[i, :i]]) for i in range(self.n_stages)]
        self.b = (D * self.n_stages)(*[float(x) for x in tab.b.double().cpu()])
        self.b_err = (D * self.n_stages)(*[float(x) for x in tab.b_err.double().cpu()])


class ERKInterpolationData(NamedTuple):
    tableau: ButcherTableau
    t0: torch.Tensor
    dt: torch.Tensor
    y0: torch.Tensor
    y1: torch.Tensor
    k: torch.Tensor


class ERKState(NamedTuple):
    tableau: ButcherTableau
    prev_vf1: Optional[torch.Tensor]


def library_tableau(method_id: int) -> ButcherTableau:
    """The Dopri5 / Tsit5 coefficients exactly as the kernels hold them."""
    D = _lib.C.c_double
    c, a, b_err, b_other, n_other = (D * 7)(), (D * 49)(), (D * 7)(), (D * 21)(), _lib.C.c_int32(0)
    _lib.check(_lib.load().tode_tableau(method_id, c, a, b_err, b_other, _lib.C.byref(n_other)), "tode_tableau")
    a_t = torch.tensor(list(a), dtype=torch.float64).reshape(7, 7)
    return ButcherTableau(
        torch.tensor(list(c), dtype=torch.float64), a_t, a_t[6].clone(), torch.tensor(list(b_err), dtype=torch.float64),
        torch.tensor(list(b_other), dtype=torch.float64).reshape(3, 7)[: n_other.value].clone(),
    )  # fmt: skip


class ExplicitRungeKutta(SingleStepMethod):
    """reference runge_kutta.py:183-282"""

    method_id = -1

    def __init__(self, term: Optional[ODETerm], tableau: ButcherTableau):
        super().__init__()
        self.term = term
        self.tableau = tableau

    def init(self, term: Optional[ODETerm], problem: InitialValueProblem, f0: Optional[torch.Tensor], *, stats: Dict[str, Any], args: Any) -> ERKState:
        prev_vf1 = None
        if self.tableau.fsal:
            term_ = term if term is not None else self.term
            assert term_ is not None
            prev_vf1 = term_.vf(problem.t_start, problem.y0, stats, args) if f0 is None else f0
        return ERKState(self.tableau, prev_vf1)

    def merge_states(self, accept: torch.Tensor, current: ERKState, previous: ERKState) -> ERKState:
        cur, prev = current.prev_vf1, previous.prev_vf1
        if cur is None or prev is None:
            return current
        _lib.require_device(accept, cur, prev)
        assert accept.element_size() == 1 and cur.dtype == prev.dtype and cur.dtype in _lib.DTYPES

        def kernel():
            a, b, mask = cur.contiguous(), prev.contiguous(), accept.contiguous()
            out = torch.empty_like(a)
            B, F = a.shape
            rc = _lib.load().tode_select_rows(_lib.DTYPES[a.dtype], B, F, _lib.ptr(mask), _lib.ptr(a), _lib.ptr(b), _lib.ptr(out), _lib.stream_of(a))
            _lib.check(rc, "tode_select_rows")
            return out

        return ERKState(current.tableau, differentiable.through(kernel, lambda a, b: differentiable.select_rows(accept, a, b), cur, prev))

    def step(self, term, running, y0, t0, dt, state: ERKState, *, stats, args):
        term_ = term if term is not None else self.term
        assert term_ is not None
        _lib.require_device(y0, t0, dt)
        assert dt.dtype == t0.dtype, "t and dt of different dtypes"
        tab = state.tableau
        h = tab.host()
        y0, t0, dt = y0.contiguous(), t0.contiguous(), dt.contiguous()
        B, F = y0.shape
        S = h.n_stages
        lib, code, stream = _lib.load(), _lib.dtype_code(y0.dtype, t0.dtype), _lib.stream_of(y0)

        vf0 = state.prev_vf1 if tab.fsal and state.prev_vf1 is not None else term_.vf(t0, y0, stats, args)
        # the slopes: one [S, B, F] array for the kernels; beside it, where gradients are wanted, the tensors as f
        # returned them (the array is filled in place, which autograd could follow only by copying it per stage)
        k = y0.new_empty((S, B, F))
        vf0 = vf0 if vf0.dtype == y0.dtype else vf0.to(y0.dtype)
        k[0].copy_(vf0.detach())
        ks = [vf0]
        y_i = y0
        for i in range(1, S):

            def stage_kernel(i=i):
                y_i, t_i = torch.empty_like(y0), torch.empty_like(t0)
                rc = lib.tode_erk_stage(code, B, F, i, h.a_rows[i], h.c[i], _lib.ptr(t0), _lib.ptr(dt), _lib.ptr(y0), _lib.ptr(k), _lib.ptr(y_i), _lib.ptr(t_i), stream)
                _lib.check(rc, "tode_erk_stage")
                return y_i, t_i

            y_i, t_i = differentiable.through(stage_kernel, partial(differentiable.stage, list(h.a_rows[i])[:i], h.c[i]), t0, dt, y0, *ks)
            k_i = term_.vf(t_i, y_i, stats, args)
            k_i = k_i if k_i.dtype == y0.dtype else k_i.to(y0.dtype)
            k[i].copy_(k_i.detach())
            ks.append(k_i)

        def combine_kernel(weights, base):
            out = torch.empty_like(y0)
            _lib.check(lib.tode_erk_combine(code, B, F, S, weights, _lib.ptr(dt), _lib.ptr(k), _lib.ptr(base), _lib.ptr(out), stream), "tode_erk_combine")
            return out

        if tab.ssal:
            y1 = y_i
        else:
            y1 = differentiable.through(partial(combine_kernel, h.b, y0), partial(differentiable.combine, list(h.b)), dt, y0, *ks)
        err = differentiable.through(
            partial(combine_kernel, h.b_err, None), lambda dt_, *ks_: differentiable.combine(list(h.b_err), dt_, None, *ks_), dt, *ks
        )

        tracked = differentiable.tracked(*ks)
        slopes = torch.stack(ks) if tracked else k  # (same values; a graph back to every evaluation of f)
        if tab.fsal:
            state = ERKState(tab, ks[-1] if tracked else k[-1])
        return StepResult(y1, err), ERKInterpolationData(tab, t0, dt, y0, y1, slopes), state, None

    def build_interpolation(self, data: ERKInterpolationData):
        raise NotImplementedError()
