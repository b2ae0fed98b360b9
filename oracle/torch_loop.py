"""TEST INFRASTRUCTURE ONLY -- never imported by the product package.

Plain-torch CPU restatement of torchode's batch-parallel adaptive explicit
Runge-Kutta solve loop for Dopri5/Tsit5 with the Integral/PID step size
controllers.  It is written as free functions over tensors (no solver classes)
and issues the *same ATen operations* (einsum, addcmul, add(alpha=), pow,
vector_norm, where, clamp) at the reference's call sites, so that on a CPU it
inherits ATen's rounding and association choices.

Only ``tests/``, ``__graft_entry__.smoke()`` and ``bench.py``'s CPU-baseline
leg may import this module, and only as a checker or as the timed baseline.

Reference sites restated (paths relative to the torchode source tree):
  * loop                    torchode/adjoints.py:50-309
  * RK step                 torchode/single_step_methods/runge_kutta.py:226-279
  * FSAL merge              torchode/single_step_methods/runge_kutta.py:216-224
  * tableaux                torchode/single_step_methods/dopri5.py:11-44,
                            torchode/single_step_methods/tsit5.py:74-114
  * Tsit5 dense weights     torchode/single_step_methods/tsit5.py:11-50
  * Tsit5 / Dopri5 quartic  torchode/single_step_methods/tsit5.py:123-139,
                            torchode/interpolation.py:138-170
  * quartic evaluation      torchode/interpolation.py:25-40,172-175
  * error ratio, PI / PID   torchode/step_size_controllers.py:170-181,289-294,
                            370-429,598-671,715-774
  * start step              torchode/step_size_controllers.py:431-490,776-835
  * f-eval counter          torchode/terms.py:41-63

Pinning status of each function is recorded next to it ("pinned by"); the
tests live in tests/test_oracle_pins.py.  The reference itself could not be
imported in the authoring container (its ``torchtyping`` dependency is absent),
so end-to-end trajectories are pinned only through the closed forms, library
special cases and reference-held examples listed there; ATen's bit-level
association is inherited, not pinned.
"""
from functools import lru_cache
from math import sqrt
from typing import Callable, Dict, NamedTuple, Optional

import torch

SUCCESS, GENERAL_ERROR, REACHED_DT_MIN, REACHED_MAX_STEPS, INFINITE_NORM = 0, 1, 2, 3, 4


# --------------------------------------------------------------------------- #
# Butcher tableaux                                                            #
# --------------------------------------------------------------------------- #


def _square(rows):
    n = len(rows)
    return [list(r) + [0.0] * (n - len(r)) for r in rows]


@lru_cache(maxsize=None)
def tsit5_dense_weights():
    """theta^2, theta^3, theta^4 monomial coefficients of Tsitouras' seven dense-output
    basis polynomials, derived the way the reference derives them (tsit5.py:11-50):
    the interpolant ``y_0 + dt * sum_s f_s b_s(t)`` is written with the factored basis
    polynomials as sympy expressions over *floating point* literals, expanded in t,
    collected by powers of t, and each coefficient converted with ``float``.  The
    intermediate products are therefore rounded by sympy's float arithmetic, and two of
    the 21 numbers differ in the last place from an exact expansion rounded once; the
    reference's solves use these.  The symbol names are the reference's, because
    sympy's canonical ordering of sums and products goes by name.

    Returns (rows for t^2, t^3, t^4; row for t^1).

    pinned by: literal equality with the kernels' and the C oracle's constants, the
    brute-force numpy.polynomial product (to 1e-14), sum_p W[p][s] == b[s], t^1 row ==
    (1,0,..,0) up to one rounding, quartic-recovery test
    (tests/interpolation_test.py:105-127).
    """
    import sympy as sp

    t, y_0, dt = sp.symbols("t y_0 dt")
    f = sp.symbols("f_1:8")
    quad = lambda p1, p0: t**2 - p1 * t + p0
    basis = [
        -1.0530884977290216 * t * (t - 1.3299890189751412) * quad(1.4364028541716351, 0.7139816917074209),
        0.1017 * t**2 * quad(2.1966568338249754, 1.2949852507374631),
        2.490627285651252793 * t**2 * quad(2.38535645472061657, 1.57803468208092486),
        -16.54810288924490272 * (t - 1.21712927295533244) * (t - 0.61620406037800089) * t**2,
        47.37952196281928122 * (t - 1.203071208372362603) * (t - 0.658047292653547382) * t**2,
        -34.87065786149660974 * (t - 1.2) * (t - 0.666666666666666667) * t**2,
        2.5 * (t - 1) * (t - 0.6) * t**2,
    ]
    powers = sp.collect(sp.expand(y_0 + dt * sum(f_s * b_s for f_s, b_s in zip(f, basis)), t), t)
    row = lambda p: [float(powers.coeff(t, p).coeff(f_s).coeff(dt)) for f_s in f]
    return [row(p) for p in (2, 3, 4)], row(1)


class Tableau(NamedTuple):
    c: torch.Tensor  # [S]    float64
    a: torch.Tensor  # [S,S]  float64
    b: torch.Tensor  # [S]
    b_err: torch.Tensor  # [S]
    b_other: torch.Tensor  # [R,S]
    name: str

    def cast(self, time_dtype, data_dtype):
        """runge_kutta.py:107-121 -- c in the time dtype, the rest in the data dtype."""
        return Tableau(
            self.c.to(time_dtype),
            self.a.to(data_dtype),
            self.b.to(data_dtype),
            self.b_err.to(data_dtype),
            self.b_other.to(data_dtype),
            self.name,
        )


def _dopri5() -> Tableau:
    """dopri5.py:11-44.  b_err = b - b_low in float64 (runge_kutta.py:84-88).

    pinned by: row sums == c, order conditions, stability / error polynomials,
    scipy.integrate RK45 coefficients.
    """
    f64 = torch.float64
    b = [35 / 384, 0, 500 / 1113, 125 / 192, -2187 / 6784, 11 / 84, 0.0]
    b_low = [1951 / 21600, 0, 22642 / 50085, 451 / 720, -12231 / 42400, 649 / 6300, 1 / 60]
    a = _square(
        [
            [],
            [1 / 5],
            [3 / 40, 9 / 40],
            [44 / 45, -56 / 15, 32 / 9],
            [19372 / 6561, -25360 / 2187, 64448 / 6561, -212 / 729],
            [9017 / 3168, -355 / 33, 46732 / 5247, 49 / 176, -5103 / 18656],
            [35 / 384, 0, 500 / 1113, 125 / 192, -2187 / 6784, 11 / 84],
        ]
    )
    mid = [
        6025192743 / 30085553152 / 2,
        0,
        51252292925 / 65400821598 / 2,
        -2691868925 / 45128329728 / 2,
        187940372067 / 1594534317056 / 2,
        -1776094331 / 19743644256 / 2,
        11237099 / 235043384 / 2,
    ]
    bt = torch.tensor(b, dtype=f64)
    return Tableau(
        torch.tensor([0.0, 1 / 5, 3 / 10, 4 / 5, 8 / 9, 1.0, 1.0], dtype=f64),
        torch.tensor(a, dtype=f64),
        bt,
        bt - torch.tensor(b_low, dtype=f64),
        torch.tensor([mid], dtype=f64),
        "dopri5",
    )


def _tsit5() -> Tableau:
    """tsit5.py:74-114.

    pinned by: row sums == c, order conditions, stability / error polynomials.
    """
    f64 = torch.float64
    b = [0.09646076681806523, 0.01, 0.4798896504144996, 1.379008574103742, -3.290069515436081, 2.324710524099774, 0.0]
    a = _square(
        [
            [],
            [0.161],
            [-0.008480655492356989, 0.335480655492357],
            [2.8971530571054935, -6.359448489975075, 4.3622954328695815],
            [5.325864828439257, -11.748883564062828, 7.4955393428898365, -0.09249506636175525],
            [5.86145544294642, -12.92096931784711, 8.159367898576159, -0.071584973281401, -0.02826905039406838],
            b[:6],
        ]
    )
    b_err = [
        0.00178001105222577714,
        0.0008164344596567469,
        -0.007880878010261995,
        0.1447110071732629,
        -0.5823571654525552,
        0.45808210592918697,
        -1 / 66,
    ]
    w, _ = tsit5_dense_weights()
    return Tableau(
        torch.tensor([0.0, 0.161, 0.327, 0.9, 0.9800255409045097, 1.0, 1.0], dtype=f64),
        torch.tensor(a, dtype=f64),
        torch.tensor(b, dtype=f64),
        torch.tensor(b_err, dtype=f64),
        torch.tensor(w, dtype=f64),
        "tsit5",
    )


TABLEAUX = {"dopri5": _dopri5(), "tsit5": _tsit5()}
ORDER = {"dopri5": 5, "tsit5": 5}


# --------------------------------------------------------------------------- #
# One explicit RK step                                                        #
# --------------------------------------------------------------------------- #


def erk_step(vf, tab: Tableau, t0, dt, y0, k0):
    """runge_kutta.py:247-272 for an FSAL+SSAL pair: returns (y1, err, k[S,B,F]).

    pinned by: linear test equation (y1 = R(z) y0, err = E(z) y0 with the
    stability / error polynomials), tests/single_step_methods_test.py:22-53.
    """
    dt_d = dt.to(dtype=y0.dtype)
    S = tab.c.shape[0]
    k = k0.new_empty((S, k0.shape[0], k0.shape[1]))
    k[0] = k0
    t_nodes = torch.addcmul(t0, tab.c[:, None], dt)
    y_i = y0
    for i in range(1, S):
        y_i = torch.einsum("j, jbf -> bf", tab.a[i, :i], k[:i])
        y_i = torch.addcmul(y0, dt_d[:, None], y_i)
        k[i] = vf(t_nodes[i], y_i)
    err = torch.einsum("b, s, sbf -> bf", dt_d, tab.b_err, k)
    return y_i, err, k


# --------------------------------------------------------------------------- #
# Step size control                                                           #
# --------------------------------------------------------------------------- #


class Controller(NamedTuple):
    """Constructor arguments of IntegralController / PIDController
    (step_size_controllers.py:263-287, 566-596)."""

    kind: str  # "integral" | "pid" | "fixed" (FixedStepController, step_size_controllers.py:116-167: needs dt0, other fields unused)
    atol: float
    rtol: float
    pcoeff: float = 0.0
    icoeff: float = 1.0
    dcoeff: float = 0.0
    dt_min: Optional[float] = None
    dt_max: Optional[float] = None
    safety: float = 0.9
    factor_min: float = 0.2
    factor_max: float = 10.0


def rms(y):
    """step_size_controllers.py:170-181."""
    return torch.linalg.vector_norm(y / sqrt(y.shape[1]), ord=2, dim=1)


def tolerances(ctrl: Controller):
    """atol/rtol are registered as torch.tensor(python_float), i.e. float32
    (step_size_controllers.py:278-279, 584-585)."""
    return torch.tensor(ctrl.atol), torch.tensor(ctrl.rtol)


def almost_zero(dtype):
    """step_size_controllers.py:251-256 / 543-548."""
    return torch.tensor(1e-5 if dtype == torch.float16 else 1e-38, dtype=dtype)


def error_ratio(ctrl: Controller, y0, y1, err):
    """step_size_controllers.py:393-401 / 738-746.

    pinned by: hand cases (atol=1, rtol=0), tests/step_size_controllers_test.py.
    """
    atol, rtol = tolerances(ctrl)
    bounds = torch.add(atol, torch.maximum(y0.abs(), y1.abs()), alpha=rtol)
    return torch.maximum(rms(err.abs() / bounds), almost_zero(y0.dtype))


def dt_factor(ctrl: Controller, order: int, ratio, prev, prev_prev):
    """step_size_controllers.py:289-294 (integral), 598-620 (PID).

    pinned by: closed form safety * ratio**(-1/order) etc. in float64.
    """
    if ctrl.kind == "integral":
        k_i = 1.0 / order
        factor = ctrl.safety * ratio ** (-k_i)
    else:
        k_i, k_p, k_d = ctrl.icoeff / order, ctrl.pcoeff / order, ctrl.dcoeff / order
        f1 = ratio ** (-(k_i + k_p + k_d))
        f2 = prev ** (k_p + 2 * k_d)
        f3 = prev_prev**-k_d
        factor = ctrl.safety * f1 * f2 * f3
    return torch.clamp(factor, min=ctrl.factor_min, max=ctrl.factor_max)


def adapt(ctrl: Controller, order: int, dt, y0, y1, err, prev, prev_prev):
    """step_size_controllers.py:370-429 / 715-774 plus update_state (663-671).

    Returns (accept, dt_next, status, ratio, prev_new, prev_prev_new).
    """
    ratio = error_ratio(ctrl, y0, y1, err)
    accept = ratio < 1.0
    dt_next = dt * dt_factor(ctrl, order, ratio, prev, prev_prev).to(dtype=dt.dtype)
    status = torch.where(torch.isfinite(ratio), SUCCESS, INFINITE_NORM)
    if ctrl.dt_min is not None or ctrl.dt_max is not None:
        lo = None if ctrl.dt_min is None else torch.tensor(ctrl.dt_min, dtype=dt.dtype)
        hi = None if ctrl.dt_max is None else torch.tensor(ctrl.dt_max, dtype=dt.dtype)
        mag = dt_next.abs()
        dt_next = torch.sign(dt_next) * torch.clamp(mag, lo, hi)
        if lo is not None:
            status = torch.where(mag < lo, REACHED_DT_MIN, status)
    if ctrl.kind == "pid":
        prev_new = torch.where(accept, ratio, prev)
        prev_prev_new = torch.where(accept, prev, prev_prev)
    else:
        prev_new, prev_prev_new = prev, prev_prev
    return accept, dt_next, status, ratio, prev_new, prev_prev_new


def initial_step(vf, ctrl: Controller, order: int, t0, y0, direction, span):
    """step_size_controllers.py:431-490 (integral) / 776-835 (PID).  The integral
    copy guards dt0 == 0 (line 481); the PID copy does not (line 826).

    pinned by: scipy.integrate._ivp.common.select_initial_step at B=1.
    """
    atol, rtol = tolerances(ctrl)
    f0 = vf(t0, y0)
    inv = torch.reciprocal(torch.add(atol, torch.abs(y0), alpha=rtol))
    d0 = rms(y0 * inv)
    d1 = rms(f0 * inv)
    tiny = torch.tensor(1e-6, dtype=d0.dtype)
    h0 = torch.where((d0 < 1e-5) | (d1 < 1e-5), tiny, 0.01 * d0 / d1)
    h0 = torch.minimum(h0, span.to(dtype=y0.dtype))
    y1 = torch.addcmul(y0, (direction * h0)[:, None], f0)
    f1 = vf(torch.addcmul(t0, direction.to(dtype=t0.dtype), h0.to(dtype=t0.dtype)), y1)
    d2 = rms((f1 - f0) * inv) / h0
    if ctrl.kind == "integral":
        d2 = torch.where(h0 == 0, torch.inf, d2)
    m = torch.maximum(d1, d2)
    h1 = torch.where(m <= 1e-15, torch.maximum(tiny, h0 * 1e-3), (0.01 / m) ** (1.0 / order))
    return (direction * torch.minimum(100 * h0, h1)).to(dtype=t0.dtype), f0


# --------------------------------------------------------------------------- #
# Dense output                                                                #
# --------------------------------------------------------------------------- #


def quartic_tsit5(tab: Tableau, dt, y0, k):
    """tsit5.py:123-139: coefficients (e, d, c, b, a), lowest power first.

    pinned by: p(0)=y0, p'(0)=dt k0, quartic recovery (5e-4).
    """
    dt_d = dt.to(dtype=y0.dtype)
    w = torch.einsum("b, cs, sbf -> cbf", dt_d, tab.b_other, k)
    return y0, dt_d[:, None] * k[0], w[0], w[1], w[2]


def quartic_dopri5(tab: Tableau, dt, y0, y1, k):
    """dopri5.py:53-60 -> interpolation.py:138-170.

    pinned by: p(0)=y0, p(1)=y1, p'(0)=dt k0, p'(1)=dt k6, p(1/2)=y_mid;
    tests/interpolation_test.py:84-102.
    """
    dt_d = dt.to(dtype=y0.dtype)
    f0 = dt_d[:, None] * k[0]
    f1 = dt_d[:, None] * k[-1]
    y_mid = y0 + torch.einsum("b, s, sbf -> bf", dt_d, tab.b_other[0], k)
    a = (2 * (f1 - f0)).add(y1 + y0, alpha=-8).add(y_mid, alpha=16)
    b = (5 * f0).add(f1, alpha=-3).add(y0, alpha=18).add(y1, alpha=14).add(y_mid, alpha=-32)
    c = f1.add(f0, alpha=-4).add(y0, alpha=-11).add(y1, alpha=-5).add(y_mid, alpha=16)
    return y0, f0, c, b, a


def quartic_eval(coeff, t0, t1, t, idx):
    """interpolation.py:25-40, 172-175: Horner on x = (t - t0) / (t1 - t0)."""
    e, d, c, b, a = (x[idx] for x in coeff)
    den = t1[idx] - t0[idx]
    den = torch.where(den.abs() > 0.0, den, 1.0)
    x = ((t - t0[idx]) / den)[:, None].to(dtype=a.dtype)
    y = a
    y = torch.addcmul(b, y, x)
    y = torch.addcmul(c, y, x)
    y = torch.addcmul(d, y, x)
    y = torch.addcmul(e, y, x)
    return y


# --------------------------------------------------------------------------- #
# The solve loop                                                              #
# --------------------------------------------------------------------------- #


def run_loop(
    y0: torch.Tensor,
    t_start: torch.Tensor,
    t_end: torch.Tensor,
    t_eval: Optional[torch.Tensor],
    dt: torch.Tensor,
    step: Callable,
    adapt: Callable,
    merge_method: Callable,
    merge_controller: Callable,
    dense: Callable,
    method_state,
    controller_state,
    *,
    max_steps: Optional[int] = None,
    on_iteration: Optional[Callable] = None,
):
    """The loop of adjoints.py:50-309 with the step method and the controller as callables:

      step(running, y, t, dt, method_state) -> (y1, interp_data, method_state_next, status | None)
      adapt(t, dt, y, y1, interp_data, controller_state) -> (accept, dt_next, controller_state_next, status | None)
      merge_method(move, new, old), merge_controller(running, new, old) -> state
      dense(interp_data) -> evaluate(t[n], idx[n]) -> [n, F]

    Returns (ys, status | None, n_steps, n_accepted, n_initialized, iterations).

    pinned by: the loop cases of tests/adjoint_test.py:26-319 restated with scripted
    callables (evaluation points hit exactly, independent stepping, several points in
    one step / on the last step, end-point evaluation, max_steps, retry after rejection,
    values stored on accept only, first-step rejection, method / controller failure,
    finished samples keep dt).
    """
    B = y0.shape[0]
    direction = torch.where(t_end > t_start, 1, -1).to(dtype=t_start.dtype)
    t, y = t_start, y0
    n_steps = torch.zeros(B, dtype=torch.long)
    n_accepted = torch.zeros(B, dtype=torch.long)
    t_min, t_max = torch.minimum(t_start, t_end), torch.maximum(t_end, t_start)
    if t_eval is not None:
        ys = y0.new_empty((B, t_eval.shape[1], y0.shape[1]))
        pending = torch.ones_like(t_eval, dtype=torch.bool)
        neg_eval = -direction[:, None] * t_eval
    neg_end = -direction * t_end
    running = torch.ones(B, dtype=torch.bool)
    dt = torch.clamp(dt, t_min - t, t_max - t)

    if t_eval is not None:
        at_start = t_eval[:, 0] == t_start
        ys[at_start, 0] = y[at_start]
        pending[at_start, 0] = False

    iterations = 0
    while True:
        iterations += 1
        y1, interp_data, method_state_next, method_status = step(running, y, t, dt, method_state)
        accept, dt_next, controller_state_next, controller_status = adapt(t, dt, y, y1, interp_data, controller_state)

        move = accept & running
        if on_iteration is not None:
            on_iteration(t, dt, accept, running, controller_state_next)
        t = torch.where(move, t + dt, t)
        y = torch.where(move[:, None], y1, y)
        method_state = merge_method(move, method_state_next, method_state)
        n_steps.add_(running)
        n_accepted.add_(move)

        running = torch.addcmul(neg_end, direction, t) < 0.0
        status = method_status
        if status is None:
            status = controller_status
        elif controller_status is not None:
            status = torch.maximum(status, controller_status)
        if max_steps is not None:
            status = torch.where(n_steps >= max_steps, REACHED_MAX_STEPS, status if status is not None else SUCCESS)
        go_on = torch.any(running)
        if status is not None:
            go_on = go_on & torch.all(status == SUCCESS)

        if t_eval is not None:
            hit = (torch.addcmul(neg_eval, direction[:, None], t[:, None]) >= 0.0) & pending
            if hit.any():
                evaluate = dense(interp_data)
                nz = hit.nonzero()
                si, ei = nz[:, 0], nz[:, 1]
                ys[si, ei] = evaluate(t_eval[si, ei], si)
                pending = torch.logical_xor(hit, pending)

        dt = torch.where(running, dt_next, dt)
        dt = torch.clamp(dt, t_min - t, t_max - t)
        controller_state = merge_controller(running, controller_state_next, controller_state)

        if bool(go_on):
            continue

        if t_eval is not None:
            n_init = torch.searchsorted(pending.int(), torch.ones((B, 1), dtype=torch.int)).squeeze(dim=1)
            return ys, status, n_steps, n_accepted, n_init, iterations
        y_end = dense(interp_data)(t_end, torch.arange(B))
        return y_end[:, None], status, n_steps, n_accepted, torch.ones(B, dtype=torch.long), iterations


def solve(
    f: Callable,
    y0: torch.Tensor,
    t_eval: Optional[torch.Tensor],
    *,
    method: str,
    controller: Controller,
    t_start: Optional[torch.Tensor] = None,
    t_end: Optional[torch.Tensor] = None,
    dt0: Optional[torch.Tensor] = None,
    max_steps: Optional[int] = None,
    trace: Optional[list] = None,
) -> Dict[str, torch.Tensor]:
    """adjoints.py:50-309 for (Dopri5|Tsit5) x (Integral|PID, rms norm): ``run_loop`` with
    the Runge-Kutta step, the error-ratio controller and the quartic dense output plugged in.

    ``f(t, y)`` is any torch callable.  Returns a dict with ys, ts, status and
    the four stats (n_f_evals is the batch-uniform CPU counter of terms.py).
    ``trace`` (optional list) receives one dict per iteration with
    t, dt, ratio, accept for localising divergences.

    pinned by: README.md:57-59 exact stats, constant-dynamics exact values
    (tests/adjoint_test.py:357-368), n_f_evals = 2 + 6 iterations, batch
    composition independence, time-reversal round trip.
    """
    if t_start is None:
        t_start = t_eval[:, 0]
    if t_end is None:
        t_end = t_eval[:, -1]
    B = y0.shape[0]
    order = ORDER[method]
    tab = TABLEAUX[method].cast(t_start.dtype, y0.dtype)
    direction_i = torch.where(t_end > t_start, 1, -1)

    calls = [0]

    def vf(t, y):
        calls[0] += 1
        return f(t, y)

    fixed = controller.kind == "fixed"
    assert not fixed or dt0 is not None, "Fixed step size solving requires you to configure dt0"
    if dt0 is None:
        dt, k0 = initial_step(vf, controller, order, t_start, y0, direction_i, (t_end - t_start).abs())
    else:
        dt, k0 = dt0, vf(t_start, y0)
    ones = torch.ones(B, dtype=y0.dtype)
    accept_all = torch.ones(B, dtype=torch.bool)

    def step(running, y, t, dt, k0):
        y1, err, k = erk_step(vf, tab, t, dt, y, k0)
        return y1, (t, dt, y, y1, err, k), k[-1], None

    def adapt_(t, dt, y, y1, data, state):
        if fixed:  # every step accepted, the next step is dt0 again, no status (step_size_controllers.py:153-163)
            return accept_all, dt0, (state[0], state[1], ones), None
        accept, dt_next, status, ratio, prev_n, prev_prev_n = adapt(controller, order, dt, y, y1, data[4], *state)
        return accept, dt_next, (prev_n, prev_prev_n, ratio), status

    def merge_method(move, new, old):
        return torch.where(move[:, None], new, old)

    def merge_controller(running, new, old):
        return torch.where(running, new[0], old[0]), torch.where(running, new[1], old[1])

    def dense(data):
        t0, dt, y, y1, _, k = data
        coeff = quartic_tsit5(tab, dt, y, k) if method == "tsit5" else quartic_dopri5(tab, dt, y, y1, k)
        return lambda tt, idx: quartic_eval(coeff, t0, t0 + dt, tt, idx)

    def on_iteration(t, dt, accept, running, state_next):
        if trace is not None:
            trace.append(dict(t=t.clone(), dt=dt.clone(), ratio=state_next[2].clone(), accept=accept.clone(), running=running.clone()))

    ys, status, n_steps, n_accepted, n_init, _ = run_loop(
        y0, t_start, t_end, t_eval, dt, step, adapt_, merge_method, merge_controller, dense, k0, (ones, ones),
        max_steps=max_steps, on_iteration=on_iteration,
    )  # fmt: skip
    if status is None:  # adjoints.py:266-270: the user always gets a status tensor
        status = torch.tensor(SUCCESS, dtype=torch.long).expand(B)
    stats = {
        "n_f_evals": torch.full((B,), calls[0], dtype=torch.long),
        "n_steps": n_steps,
        "n_accepted": n_accepted,
        "n_initialized": n_init,
    }
    ts = t_eval if t_eval is not None else t_end[:, None]
    return dict(ts=ts, ys=ys, status=status, **stats)


# --------------------------------------------------------------------------- #
# The two low-order methods: Heun 2(1) and forward Euler                      #
# --------------------------------------------------------------------------- #


def _heun() -> Tableau:
    """heun.py:10-13: c = (0, 1), a_10 = 1, b = (1/2, 1/2), low-order weights (1, 0);
    b_err = b - b_low in float64 (runge_kutta.py:84-88).  Neither FSAL nor SSAL."""
    f64 = torch.float64
    b, b_low = torch.tensor([0.5, 0.5], dtype=f64), torch.tensor([1.0, 0.0], dtype=f64)
    return Tableau(torch.tensor([0.0, 1.0], dtype=f64), torch.tensor([[0.0, 0.0], [1.0, 0.0]], dtype=f64), b, b - b_low, torch.zeros((0, 2), dtype=f64), "heun")


def erk_step_general(vf, tab: Tableau, t0, dt, y0):
    """runge_kutta.py:247-272 for a tableau that is neither FSAL nor SSAL: the first stage is evaluated anew in
    every step and y1 = y0 + sum_s (dt b_s) k_s.  Returns (y1, err, k).

    pinned by: Heun on the linear test equation, y1 = (1 + z + z^2/2) y0 and err = (z^2/2) y0."""
    dt_d = dt.to(dtype=y0.dtype)
    S = tab.c.shape[0]
    k0 = vf(t0, y0)
    k = k0.new_empty((S, k0.shape[0], k0.shape[1]))
    k[0] = k0
    t_nodes = torch.addcmul(t0, tab.c[:, None], dt)
    for i in range(1, S):
        y_i = torch.einsum("j, jbf -> bf", tab.a[i, :i], k[:i])
        y_i = torch.addcmul(y0, dt_d[:, None], y_i)
        k[i] = vf(t_nodes[i], y_i)
    y1 = y0 + torch.einsum("b, s, sbf -> bf", dt_d, tab.b, k)
    err = torch.einsum("b, s, sbf -> bf", dt_d, tab.b_err, k)
    return y1, err, k


def cubic_from_k(dt, y0, y1, k):
    """interpolation.py:84-106: Hermite cubic through (y0, y1) with end slopes k[0], k[-1]; coefficients (d, c, b, a),
    lowest power first.

    pinned by: p(0) = y0, p(1) = y1, p'(0) = dt k[0], p'(1) = dt k[-1]."""
    f0, f1 = k[0], k[-1]
    dt_d = dt.to(dtype=y0.dtype)
    y0my1 = y0 - y1
    a = torch.add(dt_d[:, None] * (f0 + f1), y0my1, alpha=2)
    b = torch.add(dt_d[:, None] * torch.add(-f1, f0, alpha=-2), y0my1, alpha=-3)
    c = dt_d[:, None] * f0
    return y0, c, b, a


def cubic_eval(coeff, t0, t1, t, idx):
    """interpolation.py:8-22, 108-111: Horner on x = (t - t0) / (t1 - t0)."""
    d, c, b, a = (x[idx] for x in coeff)
    den = t1[idx] - t0[idx]
    den = torch.where(den.abs() > 0.0, den, 1.0)
    x = ((t - t0[idx]) / den)[:, None].to(dtype=a.dtype)
    y = a
    y = torch.addcmul(b, y, x)
    y = torch.addcmul(c, y, x)
    y = torch.addcmul(d, y, x)
    return y


def linear_eval(t0, dt, y0, y1, t, idx):
    """interpolation.py:48-62: y0 + (y1 - y0) x with x = (t - t0) / dt (note: dt itself, not (t0 + dt) - t0)."""
    dy = y1 - y0
    den = dt[idx]
    den = torch.where(den.abs() > 0.0, den, 1.0)
    x = ((t - t0[idx]) / den)[:, None].to(dtype=y0.dtype)
    return torch.addcmul(y0[idx], dy[idx], x)


def solve_low_order(
    f: Callable,
    y0: torch.Tensor,
    t_eval: Optional[torch.Tensor],
    *,
    method: str,
    controller: Controller,
    t_start: Optional[torch.Tensor] = None,
    t_end: Optional[torch.Tensor] = None,
    dt0: Optional[torch.Tensor] = None,
    max_steps: Optional[int] = None,
) -> Dict[str, torch.Tensor]:
    """adjoints.py:50-309 with ``method`` "heun" (heun.py, order 2, error estimate against the Euler step, cubic dense
    output) or "euler" (euler.py, order 1, no error estimate: an adaptive controller then accepts every step and keeps
    the step size, step_size_controllers.py:382-391 / 727-736; linear dense output) and any of the three controllers.

    pinned by: the pins of the pieces above; fixed-step accuracy against the analytic solution
    (tests/fixed_step_controller_test.py:9-19), Euler's step counts [20, 16, 3] (tests/adjoint_test.py:98-118)."""
    if t_start is None:
        t_start = t_eval[:, 0]
    if t_end is None:
        t_end = t_eval[:, -1]
    B = y0.shape[0]
    heun = method == "heun"
    order = 2 if heun else 1
    tab = _heun().cast(t_start.dtype, y0.dtype)
    direction_i = torch.where(t_end > t_start, 1, -1)
    calls = [0]

    def vf(t, y):
        calls[0] += 1
        return f(t, y)

    fixed = controller.kind == "fixed"
    assert not fixed or dt0 is not None, "Fixed step size solving requires you to configure dt0"
    # (the controller's start step evaluates f twice; its f0 goes unused: neither method keeps a first-stage value)
    dt = initial_step(vf, controller, order, t_start, y0, direction_i, (t_end - t_start).abs())[0] if dt0 is None else dt0
    ones = torch.ones(B, dtype=y0.dtype)
    accept_all = torch.ones(B, dtype=torch.bool)

    def step(running, y, t, dt, state):
        if heun:
            y1, err, k = erk_step_general(vf, tab, t, dt, y)
            return y1, (t, dt, y, y1, err, k), None, None
        y1 = torch.addcmul(y, dt.to(dtype=y.dtype)[:, None], vf(t, y))
        return y1, (t, dt, y, y1, None, None), None, None

    def adapt_(t, dt, y, y1, data, state):
        if fixed:
            return accept_all, dt0, (state[0], state[1], ones), None
        if data[4] is None:  # no error estimate: accepted, step size kept, no status
            return accept_all, dt, (state[0], state[1], ones), None
        accept, dt_next, status, ratio, prev_n, prev_prev_n = adapt(controller, order, dt, y, y1, data[4], *state)
        return accept, dt_next, (prev_n, prev_prev_n, ratio), status

    def dense(data):
        t0, dt, y, y1, _, k = data
        if heun:
            coeff = cubic_from_k(dt, y, y1, k)
            return lambda tt, idx: cubic_eval(coeff, t0, t0 + dt, tt, idx)
        return lambda tt, idx: linear_eval(t0, dt, y, y1, tt, idx)

    ys, status, n_steps, n_accepted, n_init, _ = run_loop(
        y0, t_start, t_end, t_eval, dt, step, adapt_, lambda move, new, old: None,
        lambda running, new, old: (torch.where(running, new[0], old[0]), torch.where(running, new[1], old[1])),
        dense, None, (ones, ones), max_steps=max_steps,
    )  # fmt: skip
    if status is None:
        status = torch.tensor(SUCCESS, dtype=torch.long).expand(B)
    ts = t_eval if t_eval is not None else t_end[:, None]
    return dict(ts=ts, ys=ys, status=status, n_f_evals=torch.full((B,), calls[0], dtype=torch.long), n_steps=n_steps,
                n_accepted=n_accepted, n_initialized=n_init)  # fmt: skip
