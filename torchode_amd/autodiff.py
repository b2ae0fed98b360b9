"""Gradients through the solve loop itself (reference adjoints.py:33-40, 111-113, 145-147: the
reference records every torch operation of its loop; ``backprop_through_step_size_control``
decides whether the step sizes count as functions of the inputs).

Here the forward pass runs in the per-step HIP kernels (Dopri5, Tsit5) or on the operator path
(Heun, Euler) and keeps, per loop iteration, a copy of
the small loop state (t, dt, y, the FSAL derivative, the controller history, two counters).  The
backward pass walks the iterations in reverse and pulls the cotangents of the next state and of
the evaluation points back through each, with the accept / running / evaluation decisions taken
from the record.  For Dopri5 / Tsit5 one iteration is reversed by HIP kernels
(``reverse_sweep_kernels``: the stage values are recomputed by the forward stage kernel and ``f``,
everything after the stages -- dense output, state update, step clamp, controller, error ratio --
is one reverse kernel, each stage another; only ``f``'s own vector-Jacobian products are
autograd's).  ``reverse_sweep_torch`` restates the iteration as differentiable torch operations
instead (Heun and Euler, and the checker of the kernels in the tests).  Either way ``f`` is
evaluated six times per iteration again.  Memory: one state copy per iteration instead of the
reference's whole operation graph.

Gradients flow to ``y0``, to the parameters of the term, to the tensors inside ``args`` (a
tensor, or tuples / lists / dicts of them) and to the times (``t_start``, ``t_end``, ``t_eval``,
a user's ``dt0``): the start of the loop, the clamp of every step to the time range and the
position of an evaluation point inside its step are functions of them, as in the reference,
while which step passes which point is a recorded decision.
"""
from math import sqrt
from typing import Any, List, Optional, Sequence

import torch

from . import _lib
from .problems import InitialValueProblem
from .single_step_methods import Euler, Heun


def tensor_leaves(obj) -> List[torch.Tensor]:
    """The tensors inside ``obj``: a tensor itself, or tuples, lists and dicts (by value) of such."""
    if isinstance(obj, torch.Tensor):
        return [obj]
    if isinstance(obj, (tuple, list)):
        return [t for item in obj for t in tensor_leaves(item)]
    if isinstance(obj, dict):
        return [t for item in obj.values() for t in tensor_leaves(item)]
    return []


def map_tensors(obj, fn):
    """``obj`` with ``fn`` applied to the tensors that ``tensor_leaves`` finds; containers are rebuilt."""
    if isinstance(obj, torch.Tensor):
        return fn(obj)
    if isinstance(obj, tuple):
        return tuple(map_tensors(item, fn) for item in obj)
    if isinstance(obj, list):
        return [map_tensors(item, fn) for item in obj]
    if isinstance(obj, dict):
        return {key: map_tensors(item, fn) for key, item in obj.items()}
    return obj


def captured_leaves(term, problem: InitialValueProblem, args) -> List[torch.Tensor]:
    """Leaf tensors that require grad and that ``f(t_start, y0)`` depends on without their being an argument of it:
    what ``f`` closes over, and parameters or buffers of a module behind it (directly, or through tensors computed
    from them).  Found by evaluating ``f`` once on detached inputs under grad mode and walking the graph of the result.
    The reference's loop is torch operations throughout, so autograd reaches such tensors by itself
    (adjoints.py:135-260); here they have to be named as differentiation targets of the reverse sweep."""
    from .builtin_terms import BuiltinTerm

    f = getattr(term, "f", None)
    found, y = [], None
    plain_term = not term._parameters and not term._buffers and len(term._modules) == 1
    if plain_term and isinstance(f, BuiltinTerm) and type(f).__module__ == BuiltinTerm.__module__ and not f._modules:
        # a plain term around one of the library's built-in right-hand sides, which compute from their own buffers and
        # parameters alone: the walk starts at those, without an evaluation of f
        held = [x for x in list(f._buffers.values()) + list(f._parameters.values()) if x is not None and x.requires_grad]
        found = [x for x in held if x.is_leaf]
        stack = [x.grad_fn for x in held if not x.is_leaf]
    else:
        with torch.enable_grad():
            y = problem.y0.detach().requires_grad_()
            t = problem.t_start.detach()
            # (args reaches f by identity, reference tests/extra_args_test.py:16-22; only tensors in it that require
            # grad are swapped for detached ones, so that the walk stops at them: the caller names those itself)
            plain_args = map_tensors(args, lambda a: a.detach()) if any(a.requires_grad for a in tensor_leaves(args)) else args
            out = term.f(t, y, plain_args) if term.with_args else term.f(t, y)
        stack = [getattr(out, "grad_fn", None)]
    seen = set()
    while stack:
        fn = stack.pop()
        if fn is None or fn in seen:
            continue
        seen.add(fn)
        var = getattr(fn, "variable", None)  # AccumulateGrad nodes hold the leaf
        if var is not None and var is not y and var.requires_grad and not any(var is v for v in found):
            found.append(var)
        stack.extend(nxt for nxt, _ in fn.next_functions)
    return found


def wants_grad_through_term(term, problem: InitialValueProblem, args, probe: bool = True) -> bool:
    """True if a solve under grad mode has to be differentiable because of the term alone: a parameter or buffer of
    it, a tensor in ``args``, or (looked for only with ``probe``, since it takes an evaluation of ``f``) a tensor its
    ``f`` closes over requires grad."""
    from .builtin_terms import BuiltinTerm

    f = getattr(term, "f", None)
    if isinstance(f, BuiltinTerm) and not term._parameters and not term._buffers and len(term._modules) == 1:
        # the common fast case, without nn.Module's recursive iterators: a plain term around a built-in right-hand
        # side, which holds all it uses as its own buffers
        if any(b is not None and b.requires_grad for b in f._buffers.values()) or any(p is not None and p.requires_grad for p in f._parameters.values()):
            return True
        return bool(args is not None and any(a.requires_grad for a in tensor_leaves(args)))
    if isinstance(term, torch.nn.Module) and (any(p.requires_grad for p in term.parameters()) or any(b.requires_grad for b in term.buffers())):
        return True
    if any(a.requires_grad for a in tensor_leaves(args)):
        return True
    if not probe or f is None or isinstance(f, BuiltinTerm):  # (a built-in term holds all it uses as buffers)
        return False
    return bool(captured_leaves(term, problem, args))


class LoopRecord:
    """State before each iteration (and after the last): what the forward pass hands to the backward pass."""

    FIELDS = ("t", "dt", "y", "k0", "prev", "pprev", "running", "n_accepted")

    def __init__(self):
        self.states: List[tuple] = []
        self.iterations = 0  # set by the forward pass when the loop has stopped
        self.arrays = None  # the same record as entry-major arrays, where the whole-solve kernel wrote it
        self.flags = None  # that kernel's flag words, still on the device

    def snapshot(self, t, dt, y, k0, hist, ints):
        self.states.append((t.clone(), dt.clone(), y.clone(), k0.clone(), hist[0].clone(), hist[1].clone(), ints[0].clone(), ints[3].clone()))

    def snapshot_protocol(self, t, dt, y, controller_state, running, n_accepted):
        """The same record from the operator path: a method without a first-same-as-last slope has nothing to carry
        (zeros stand in), and only the PID controller carries error ratios."""
        ones = torch.ones_like(y[:, 0])
        prev = getattr(controller_state, "prev_error_ratio", ones)
        pprev = getattr(controller_state, "prev_prev_error_ratio", ones)
        self.states.append((t.clone(), dt.clone(), y.clone(), torch.zeros_like(y), prev.clone(), pprev.clone(), running.clone(), n_accepted.clone()))

    def any_point_written(self, problem: InitialValueProblem) -> bool:
        """Whether an iteration of the recorded loop passed an evaluation point that was still to be written
        (adjoints.py:215-234): the last recorded time against the points, the one at ``t_start`` aside."""
        t_last = self.arrays["t"][self.iterations] if self.arrays is not None and not self.states else self.states[-1][0]
        direction = torch.where(problem.t_end > problem.t_start, 1.0, -1.0).to(t_last.dtype)[:, None]
        passed = direction * t_last[:, None] >= direction * problem.t_eval
        passed[:, 0] &= problem.t_eval[:, 0] != problem.t_start
        return bool(passed.any())

    def trimmed(self, iterations: int) -> List[dict]:
        """States 0..iterations; iterations enqueued after the batch had stopped changed nothing."""
        if not self.states and self.arrays is not None:  # (views of the arrays, made when a per-iteration sweep asks)
            self.states = [tuple(self.arrays[k][i] for k in self.FIELDS) for i in range(self.arrays["t"].shape[0])]
            return [dict(zip(self.FIELDS, s)) for s in self.states[: iterations + 1]]
        states = self.states[:iterations] + [self.states[-1]]
        return [dict(zip(self.FIELDS, s)) for s in states]


class Replay:
    """One loop iteration (and the start of the loop) as differentiable torch operations."""

    def __init__(self, method, controller, term, args, problem: InitialValueProblem, through_control: bool, dt0=None):
        if isinstance(method, Euler):  # (reference euler.py:29-56: one slope, no error estimate, linear dense output)
            self.a, self.c, self.b, self.b_err = [[]], [0.0], [1.0], None
            self.fsal = self.ssal = False
            self.dense_kind = "linear"
        else:
            tab = method.tableau
            self.a = [[float(x) for x in row] for row in tab.a.tolist()]
            self.c = [float(x) for x in tab.c.tolist()]
            self.b = [float(x) for x in tab.b.tolist()]
            self.b_err = [float(x) for x in tab.b_err.tolist()]
            self.fsal, self.ssal = bool(tab.fsal), bool(tab.ssal)
            if isinstance(method, Heun):
                self.dense_kind = "cubic"
            else:
                self.b_other = [[float(x) for x in row] for row in tab.b_other.tolist()]
                self.dense_kind = "tsit5" if method.method_id == _lib.TSIT5 else "dopri5"
        self.n_stages = len(self.c)
        self.order = float(method.convergence_order())
        c = controller.c_struct()
        self.pid = c.kind == _lib.CTRL_PID
        # fixed steps (reference step_size_controllers.py:116-167): every step accepted, the next step is dt0 again
        self.fixed, self.dt0 = c.kind == _lib.CTRL_FIXED, dt0
        self.atol, self.rtol = float(c.atol), float(c.rtol)
        self.safety, self.fmin, self.fmax = float(c.safety), float(c.factor_min), float(c.factor_max)
        self.dt_min = float(c.dt_min) if c.has_dt_min else None
        self.dt_max = float(c.dt_max) if c.has_dt_max else None
        if self.pid:
            k_i, k_p, k_d = c.icoeff / self.order, c.pcoeff / self.order, c.dcoeff / self.order
            self.e1, self.e2, self.e3 = -(k_i + k_p + k_d), k_p + 2 * k_d, -k_d
        else:
            self.e1, self.e2, self.e3 = -1.0 / self.order, 0.0, 0.0
        self.term, self.args = term, args
        self.through_control = through_control
        self.t_start, self.t_end, self.t_eval = problem.t_start, problem.t_end, problem.t_eval
        self._direction = None

    @property
    def direction(self):
        if self._direction is None:  # (formed when a sweep in torch operations asks for it)
            self._direction = torch.where(self.t_end > self.t_start, 1.0, -1.0).to(self.t_start.dtype)
        return self._direction

    # the ends of the time range are functions of t_start and t_end: formed where they are used, so that every
    # iteration of the reverse sweep differentiates a graph of its own
    @property
    def fixed_dt(self):
        """The step a fixed-step controller hands back every time: the user's ``dt0`` itself, so with
        ``through_control`` its gradient collects a share from every step."""
        if not self.fixed:
            return None
        dt = self.dt0.to(self.t_start.dtype)
        return dt if self.through_control else dt.detach()

    @property
    def t_lo(self):
        return torch.minimum(self.t_start, self.t_end)

    @property
    def t_hi(self):
        return torch.maximum(self.t_end, self.t_start)

    def f(self, t, y):
        out = self.term.f(t, y, self.args) if self.term.with_args else self.term.f(t, y)
        return out if out.dtype == y.dtype else out.to(y.dtype)  # (as the forward pass takes what f returns)

    def rms(self, x):
        return torch.linalg.vector_norm(x / sqrt(x.shape[1]), ord=2, dim=1)

    # ---- reference step_size_controllers.py:431-490 / 776-835 ----
    def first_step(self, y0, f0):
        inv = 1.0 / (self.atol + self.rtol * y0.abs())
        d0, d1 = self.rms(y0 * inv), self.rms(f0 * inv)
        small = (d0 < 1e-5) | (d1 < 1e-5)
        h0 = torch.where(small, torch.full_like(d0, 1e-6), 0.01 * d0 / torch.where(small, torch.ones_like(d1), d1))
        h0 = torch.minimum(h0, (self.t_end - self.t_start).abs().to(h0.dtype))
        step = (self.direction.to(h0.dtype) * h0)
        f1 = self.f(self.t_start + step.to(self.t_start.dtype), y0 + step[:, None] * f0)
        d2 = self.rms((f1 - f0) * inv) / h0
        if not self.pid:
            d2 = torch.where(h0 == 0, torch.full_like(d2, float("inf")), d2)
        m = torch.maximum(d1, d2)
        tiny = m <= 1e-15
        h1 = torch.where(tiny, torch.clamp_min(h0 * 1e-3, 1e-6), (0.01 / torch.where(tiny, torch.ones_like(m), m)) ** (1.0 / self.order))
        return (self.direction.to(h0.dtype) * torch.minimum(100 * h0, h1)).to(self.t_start.dtype)

    # ---- reference runge_kutta.py:226-279, step_size_controllers.py:370-429 / 715-774, adjoints.py:150-255 ----
    def attempt(self, state: dict):
        """The step from ``state`` and the controller's view of it: stage derivatives, y1, error ratio
        and the step size it proposes."""
        t, dt, y, k0, prev, pprev = (state[k] for k in ("t", "dt", "y", "k0", "prev", "pprev"))
        dtd = dt.to(y.dtype)
        S = self.n_stages
        ks = [k0 if self.fsal else self.f(t, y)]
        yi = y
        for i in range(1, S):
            s = sum(self.a[i][j] * ks[j] for j in range(i) if self.a[i][j] != 0.0)
            yi = y + dtd[:, None] * s
            ks.append(self.f(t + self.c[i] * dt, yi))
        y1 = yi if self.ssal else y + dtd[:, None] * sum(self.b[s] * ks[s] for s in range(S) if self.b[s] != 0.0)
        if self.fixed_dt is not None:
            return ks, y1, None, self.fixed_dt
        if self.b_err is None:  # no error estimate: the controllers accept and keep the step size
            return ks, y1, None, dt
        err = dtd[:, None] * sum(self.b_err[s] * ks[s] for s in range(S) if self.b_err[s] != 0.0)
        scale = self.atol + self.rtol * torch.maximum(y.abs(), y1.abs())
        ratio = torch.clamp_min(self.rms(err.abs() / scale), 1e-38)
        factor = self.safety * ratio**self.e1
        if self.pid:
            if self.e2 != 0.0:
                factor = factor * prev**self.e2
            if self.e3 != 0.0:
                factor = factor * pprev**self.e3
        dt_next = dt * factor.clamp(self.fmin, self.fmax).to(dt.dtype)
        if self.dt_min is not None or self.dt_max is not None:
            dt_next = torch.sign(dt_next) * dt_next.abs().clamp(self.dt_min, self.dt_max)
        if not self.through_control:
            dt_next = dt_next.detach()
        return ks, y1, ratio, dt_next

    def advance(self, state: dict, attempt, accept, running_new, hits):
        """The loop's update with the decisions given: the next state's differentiable part, and the
        dense-output values at ``hits`` = (samples, points)."""
        t, dt, y, k0, prev, pprev, running = (state[k] for k in ("t", "dt", "y", "k0", "prev", "pprev", "running"))
        ks, y1, ratio, dt_next = attempt
        move = accept & running
        y_new = torch.where(move[:, None], y1, y)
        k0_new = torch.where(move[:, None], ks[-1], k0) if self.fsal else k0
        t_new = torch.where(move, t + dt, t)
        dt_new = torch.where(running_new, dt_next, dt)
        dt_new = torch.clamp(dt_new, self.t_lo - t_new, self.t_hi - t_new)  # (reference adjoints.py:251; its tie rules differ from minimum / maximum)
        keep = running_new & accept
        shift = self.pid and ratio is not None
        prev_new, pprev_new = (torch.where(keep, ratio, prev), torch.where(keep, prev, pprev)) if shift else (prev, pprev)

        values = None
        if hits is not None:
            rows, points = hits
            at = self.t_eval[rows, points] if points is not None else self.t_end[rows]
            values = self.dense(t[rows], dt[rows], y[rows], y1[rows], [k[rows] for k in ks], at)
        return (y_new, k0_new, t_new, dt_new, prev_new, pprev_new), values

    def iteration(self, state: dict, accept, running_new, hits):
        return self.advance(state, self.attempt(state), accept, running_new, hits)

    # ---- reference tsit5.py:123-139, dopri5.py:53-60, interpolation.py:25-40, 138-170 ----
    def dense(self, t0, dt, y0, y1, ks, at):
        h = dt.to(y0.dtype)[:, None]
        if self.dense_kind == "linear":  # reference interpolation.py:48-60: the step size itself divides
            den = torch.where(dt.abs() > 0, dt, torch.ones_like(dt))
            return y0 + (y1 - y0) * ((at - t0) / den).to(y0.dtype)[:, None]
        weighted = lambda w: h * sum(w[s] * ks[s] for s in range(7) if w[s] != 0.0)
        if self.dense_kind == "cubic":  # Hermite cubic from the first and last slope, reference interpolation.py:84-106
            f0, f1, gap = ks[0], ks[-1], y0 - y1
            q = [y0, h * f0, torch.add(h * torch.add(-f1, f0, alpha=-2), gap, alpha=-3), torch.add(h * (f0 + f1), gap, alpha=2)]
        elif self.dense_kind == "tsit5":
            q = [y0, h * ks[0], weighted(self.b_other[0]), weighted(self.b_other[1]), weighted(self.b_other[2])]
        else:
            # (the reference's chains of add(alpha=...), interpolation.py:152-166: one rounding per term, so that where
            # the terms cancel to the last unit the remainder is the forward pass's)
            f0, f1, mid = h * ks[0], h * ks[6], y0 + weighted(self.b_other[0])
            q = [
                y0,
                f0,
                f1.add(f0, alpha=-4).add(y0, alpha=-11).add(y1, alpha=-5).add(mid, alpha=16),
                (5 * f0).add(f1, alpha=-3).add(y0, alpha=18).add(y1, alpha=14).add(mid, alpha=-32),
                (2 * (f1 - f0)).add(y1 + y0, alpha=-8).add(mid, alpha=16),
            ]
        den = (t0 + dt) - t0
        den = torch.where(den.abs() > 0, den, torch.ones_like(den))
        x = ((at - t0) / den).to(y0.dtype)[:, None]
        out = q[-1]
        for p in range(len(q) - 2, -1, -1):
            out = out * x + q[p]
        return out


def simulate_hits(replay: Replay, states: Sequence[dict], n_eval: int):
    """Which evaluation points each iteration wrote (adjoints.py:215-234), from the recorded times:
    a list of (samples, points) index pairs, None where an iteration wrote nothing."""
    if n_eval == 0:
        return [None] * (len(states) - 2) + [(torch.arange(states[0]["t"].shape[0], device=states[0]["t"].device), None)]
    t_eval, direction = replay.t_eval, replay.direction
    pending = torch.ones_like(t_eval, dtype=torch.bool)
    pending[:, 0] = t_eval[:, 0] != replay.t_start
    hits = []
    for n in range(len(states) - 1):
        t_new = states[n + 1]["t"]
        passed = direction[:, None] * t_new[:, None] >= direction[:, None] * t_eval
        hit = pending & passed
        pending = pending & ~hit
        idx = hit.nonzero()
        hits.append((idx[:, 0], idx[:, 1]) if idx.shape[0] > 0 else None)
    return hits


STATE_NAMES = ("y", "k0", "t", "dt", "prev", "pprev")
LAST_SWEEP = None  # "kernels" or "torch": what the most recent backward pass went through


def _add(total, part):
    return part if total is None else (total if part is None else total + part)


def reverse_sweep_torch(replay: Replay, states, hits, grad_ys, params):
    """The iterations in reverse, each restated as torch operations (Replay.iteration) and differentiated by
    autograd.  Returns the cotangents of the state before the first iteration and the gradients of ``params``."""
    names = STATE_NAMES
    add = _add
    adj = {k: None for k in names}
    grad_params = [None] * len(params)
    for n in range(len(states) - 2, -1, -1):
        now, then = states[n], states[n + 1]
        accept = (then["n_accepted"] - now["n_accepted"]) > 0
        live = dict(now, running=now["running"] != 0)
        with torch.enable_grad():
            for k in names:
                live[k] = now[k].detach().requires_grad_()
            outs, values = replay.iteration(live, accept, then["running"] != 0, hits[n])
            targets, cotangents = [], []
            for k, out in zip(names, outs):
                if adj[k] is not None and out.requires_grad:
                    targets.append(out)
                    cotangents.append(adj[k])
            if values is not None:
                rows, points = hits[n]
                targets.append(values)
                cotangents.append(grad_ys[rows, points] if points is not None else grad_ys[rows, 0])
            if not targets:
                adj = {k: None for k in names}
                continue
            wrt = [live[k] for k in names] + params
            grads = torch.autograd.grad(targets, wrt, cotangents, allow_unused=True, retain_graph=True)
        adj = dict(zip(names, grads[: len(names)]))
        for i, g in enumerate(grads[len(names) :]):
            grad_params[i] = add(grad_params[i], g)

    return adj, grad_params


def reverse_sweep_whole(adjoint, replay: Replay, term, problem, dt0, record, grad_ys, params):
    """All iterations in reverse in one kernel (tode_solve_builtin_backward): for a built-in term whose forward pass
    left its record in entry-major arrays.  The right-hand side and its vector-Jacobian product are evaluated in the
    kernel; what comes back are the cotangents of the state before the first iteration and of the term's per-sample
    parameter table, which autograd carries on to the tensors the table was made from."""
    lib = _lib.load()
    f = term.f
    method, controller = adjoint.step_method, adjoint.step_size_controller
    ctrl = controller.c_struct()
    y0 = problem.y0
    B, F = y0.shape
    E = problem.n_evaluation_points
    dev, dtype = y0.device, y0.dtype
    new = lambda *shape, dt=dtype: torch.empty(shape, dtype=dt, device=dev)
    zeros = lambda *shape, dt=dtype: torch.zeros(shape, dtype=dt, device=dev)
    contiguous = lambda x: x.detach().to(dtype).contiguous()
    # (t_start / t_end are usually columns of t_eval: handed over with their strides, unless their gradients are wanted)
    strided = lambda x: x.detach() if (x.dtype == dtype and x.stride(0) >= 1 and not x.requires_grad) else contiguous(x)
    t_start, t_end = strided(replay.t_start), strided(replay.t_end)
    t_eval = None if replay.t_eval is None else contiguous(replay.t_eval)
    L, arrays = record.iterations, record.arrays

    # Which iteration wrote which evaluation point (adjoints.py:215-234: the first whose new time has passed it), and
    # each sample's points ordered by it: worked out by the library from the record's times, in two kernels in front
    # of the sweep.  The same in torch operations, handed in, for the tests to hold against that.
    iterations_sorted = points_by_iteration = None
    if E > 0 and getattr(adjoint, "backward_points_in_torch", False):
        direction = torch.where(t_end > t_start, 1.0, -1.0).to(dtype)
        reached = (direction[None, :] * arrays["t"][1 : L + 1]).t().contiguous()  # [B, L], ascending
        hit = torch.searchsorted(reached, direction[:, None] * t_eval) if L > 0 else torch.zeros((B, E), dtype=torch.long, device=dev)
        hit = torch.where(hit < L, hit, torch.full_like(hit, -1))
        hit[:, 0] = torch.where(t_eval[:, 0] == t_start, torch.full_like(hit[:, 0], -1), hit[:, 0])
        iterations_sorted, points_by_iteration = torch.sort(hit.to(torch.int32), dim=1, stable=True)
        iterations_sorted, points_by_iteration = iterations_sorted.contiguous(), points_by_iteration.to(torch.int32).contiguous()
    wants = lambda x: x is not None and x.requires_grad
    g_t_start = zeros(B) if wants(replay.t_start) else None
    g_t_end = zeros(B) if wants(replay.t_end) else None
    g_t_eval = zeros(B, E) if (E > 0 and wants(replay.t_eval)) else None

    with torch.no_grad():
        par = f.builtin_params().detach().to(device=dev, dtype=dtype).contiguous()
    P = par.shape[1]
    scal = list(getattr(f, "builtin_scalars", lambda: ())()) + [0.0] * 4
    a = _lib.SolveArgs()
    a.dtype, a.method, a.term, a.n_features, a.n_eval, a.n_params, a.batch = _lib.DTYPES[dtype], method.method_id, f.builtin_kind, F, E, P, B
    a.max_steps, a.iteration_cap = -1, -1
    a.term_scalars = (_lib.C.c_double * 4)(*scal[:4])
    a.t_start, a.t_end, a.t_start_stride, a.t_end_stride = t_start.data_ptr(), t_end.data_ptr(), t_start.stride(0), t_end.stride(0)
    a.t_eval, a.params = _lib.ptr(t_eval), (par.data_ptr() if par.numel() else None)
    names = ("t", "dt", "y", "k0", "prev", "pprev", "running", "n_accepted")
    rec = _lib.SolveRecord(arrays["t"].shape[0], *(arrays[k].data_ptr() for k in names))
    a.record = _lib.C.addressof(rec)

    out_y, out_k0 = new(B, F), new(B, F)
    out_s = new(4, B)
    g_par = new(B, max(P, 1))
    grad = grad_ys.detach().to(dtype).contiguous()
    scratch = torch.empty(max(lib.tode_solve_backward_scratch_bytes(_lib.C.byref(a)), 1), dtype=torch.uint8, device=dev)
    ad = _lib.SolveAdjoint()
    ad.grad_ys, ad.iterations, ad.through_control = grad.data_ptr(), L, int(bool(replay.through_control))
    # the start of the loop in the kernel too, unless a time wants a gradient (the kernel takes the times of that part
    # as constants): what comes back is then the cotangent of y0 itself
    through_start = getattr(adjoint, "backward_start_in_kernel", True) and not any(wants(x) for x in (replay.t_start, replay.t_end, replay.t_eval, dt0))
    ad.through_start = int(through_start)
    if dt0 is not None:
        a.dt0 = dt0.data_ptr()  # (not read: it says that the first step was given)
    ad.scratch, ad.scratch_bytes = scratch.data_ptr(), scratch.numel()
    ad.points_by_iteration, ad.iterations_sorted = _lib.ptr(points_by_iteration), _lib.ptr(iterations_sorted)
    ad.a_y, ad.a_k0 = out_y.data_ptr(), out_k0.data_ptr()
    ad.a_t, ad.a_dt, ad.a_prev, ad.a_pprev = (out_s[i].data_ptr() for i in range(4))
    ad.g_params = g_par.data_ptr()
    ad.g_t_start, ad.g_t_end, ad.g_t_eval = _lib.ptr(g_t_start), _lib.ptr(g_t_end), _lib.ptr(g_t_eval)
    rc = lib.tode_solve_builtin_backward(_lib.C.byref(a), _lib.C.byref(ctrl), _lib.C.byref(ad), _lib.stream_of(y0))
    if rc == _lib.E_UNSUPPORTED:
        return None  # (a shape the one-kernel sweep is not built for: the caller takes the per-iteration kernels)
    _lib.check(rc, "tode_solve_builtin_backward")

    # the parameter table is a function of the term's tensors (a reshape, a negation ...): autograd takes its cotangent on
    grad_params = [None] * len(params)
    if params and P > 0:
        with torch.enable_grad():
            f.__dict__.pop("_params_view", None)  # (a table kept from a call without grad mode has no graph)
            table = f.builtin_params()
            f.__dict__.pop("_params_view", None)
            if table.requires_grad:
                grads = torch.autograd.grad(table, params, g_par[:, :P].to(table.dtype), allow_unused=True)
                grad_params = list(grads)
    for given, collected in ((replay.t_start, g_t_start), (replay.t_end, g_t_end), (replay.t_eval, g_t_eval)):
        if collected is None:
            continue
        for j, q in enumerate(params):
            if q is given:
                grad_params[j] = _add(grad_params[j], collected.to(q.dtype))
                break
    adj = dict(y=out_y, k0=out_k0, t=out_s[0], dt=out_s[1], prev=out_s[2], pprev=out_s[3], through_start=through_start)
    return adj, grad_params


def reverse_sweep_kernels(adjoint, replay: Replay, term, args, problem, dt0_given, dt0, states, hits, grad_ys, params, params_given):
    """The iterations in reverse through the library's reverse kernels (tode_step_finish_backward,
    tode_step_stage_backward): per iteration the stage values are recomputed by the forward stage kernel and ``f``
    (six evaluations under grad mode, each a small graph of its own), the finish kernel is reversed in one launch,
    and each stage in one launch after the vector-Jacobian product of ``f`` that autograd supplies.  Same result as
    ``reverse_sweep_torch`` (the tests compare the two)."""
    lib = _lib.load()
    method, controller = adjoint.step_method, adjoint.step_size_controller
    ctrl = controller.c_struct()
    cref = _lib.C.byref(ctrl)
    y0 = problem.y0
    B, F = y0.shape
    E = problem.n_evaluation_points
    dev, dtype, ttype = y0.device, y0.dtype, replay.t_start.dtype
    stream = _lib.stream_of(y0)
    new = lambda *shape, dt=dtype: torch.empty(shape, dtype=dt, device=dev)
    zeros = lambda *shape, dt=dtype: torch.zeros(shape, dtype=dt, device=dev)
    contiguous = lambda x, dt: x.detach().to(dt).contiguous()
    t_start, t_end = contiguous(replay.t_start, ttype), contiguous(replay.t_end, ttype)
    t_eval = None if replay.t_eval is None else contiguous(replay.t_eval, ttype)
    fixed = ctrl.kind == _lib.CTRL_FIXED
    fixed_dt = contiguous(dt0, ttype) if fixed else None
    n_iterations = len(states) - 1

    # which iteration wrote which evaluation point
    hit_iteration = None
    if E > 0:
        hit_iteration = torch.full((B, E), -1, dtype=torch.int32, device=dev)
        for n, h in enumerate(hits):
            if h is not None:
                hit_iteration[h[0], h[1]] = n
    grad_ys = contiguous(grad_ys, dtype)

    # gradients of the times, collected by the kernels
    wants = lambda x: x is not None and x.requires_grad
    g_t_start = zeros(B, dt=ttype) if wants(replay.t_start) else None
    g_t_end = zeros(B, dt=ttype) if wants(replay.t_end) else None
    g_t_eval = zeros(B, E, dt=ttype) if (E > 0 and wants(replay.t_eval)) else None
    g_fixed_dt = zeros(B, dt=ttype) if (fixed and wants(dt0) and replay.through_control) else None

    # a scratch state for the forward stage kernel (it reads t, dt, y and the k's, and writes ystage / tnode)
    st = _lib.StepState()
    st.dtype, st.time_dtype, st.method, st.n_features, st.n_eval = _lib.DTYPES[dtype], _lib.DTYPES[ttype], method.method_id, F, 0
    st.batch, st.max_steps = B, -1
    clear = zeros(_lib.STEP_FLAG_WORDS, dt=torch.int32)
    idle = zeros(B, dt=torch.int32)
    st.flags = clear.data_ptr()
    st.fixed_dt = _lib.ptr(fixed_dt)
    st.t_start, st.t_end = t_start.data_ptr(), t_end.data_ptr()
    for name in ("running", "cursor", "n_steps", "n_accepted", "status", "monotone"):
        setattr(st, name, idle.data_ptr())
    sref = _lib.C.byref(st)

    ad = _lib.StepAdjoint()
    ad.dtype, ad.time_dtype, ad.method, ad.n_features, ad.n_eval = st.dtype, st.time_dtype, st.method, F, E
    ad.batch, ad.through_control = B, int(bool(replay.through_control))
    ad.t_start, ad.t_end, ad.t_eval = t_start.data_ptr(), t_end.data_ptr(), _lib.ptr(t_eval)
    ad.fixed_dt, ad.hit_iteration, ad.grad_ys = _lib.ptr(fixed_dt), _lib.ptr(hit_iteration), grad_ys.data_ptr()
    ad.g_t_start, ad.g_t_end, ad.g_t_eval, ad.g_fixed_dt = _lib.ptr(g_t_start), _lib.ptr(g_t_end), _lib.ptr(g_t_eval), _lib.ptr(g_fixed_dt)
    aref = _lib.C.byref(ad)

    g_k = new(7, B, F)
    g_y, g_y1 = new(B, F), new(B, F)
    g_t, g_dt = new(B, dt=ttype), new(B, dt=ttype)
    g_hist = new(2, B)
    for i in range(7):
        ad.g_k[i] = g_k[i].data_ptr()
    ad.g_y, ad.g_y1, ad.g_t, ad.g_dt, ad.g_prev, ad.g_pprev = (x.data_ptr() for x in (g_y, g_y1, g_t, g_dt, g_hist[0], g_hist[1]))

    f, with_args = term.f, term.with_args

    def rhs(tt, yy):
        out = f(tt, yy, args) if with_args else f(tt, yy)
        if out.dtype != dtype or not out.is_contiguous() or out.shape != yy.shape:
            out = out.to(dtype).expand(yy.shape).contiguous()
        return out

    adj = None  # cotangents of the state after the iteration at hand: (y, k0, t, dt, prev, pprev) or None for zeros
    grad_params = [None] * len(params)
    last = n_iterations - 1
    for n in range(last, -1, -1):
        has_hits = hits[n] is not None if E > 0 else n == last
        if adj is None and not has_hits:
            continue
        now, then = states[n], states[n + 1]
        moved = ((then["n_accepted"] - now["n_accepted"]) > 0).to(torch.int32)
        running_next = (then["running"] != 0).to(torch.int32)
        # ---- the stages again: forward kernels and f, keeping f's graphs ----
        st.t, st.dt, st.y, st.k0 = (now[k].data_ptr() for k in ("t", "dt", "y", "k0"))
        st.y0, st.ys = now["y"].data_ptr(), now["y"].data_ptr()  # (not used by the stage kernel)
        st.ratio_prev, st.ratio_pprev = now["prev"].data_ptr(), now["pprev"].data_ptr()
        st.k[0] = now["k0"].data_ptr()
        ks, inputs = [now["k0"]], [None]
        for i in range(1, 7):
            yi, ti = new(B, F), new(B, dt=ttype)
            st.ystage[i], st.tnode = yi.data_ptr(), ti.data_ptr()
            _lib.check(lib.tode_step_stage(sref, cref, i, stream), "tode_step_stage")
            with torch.enable_grad():
                yi.requires_grad_()
                ti.requires_grad_()
                ki = rhs(ti, yi)
            kd = ki.detach()
            ks.append(kd)
            inputs.append((yi, ti, ki))
            st.k[i] = kd.data_ptr()
        # ---- everything after the stages, reversed ----
        ad.iteration, ad.end_point = n, int(E == 0 and n == last)
        ad.t, ad.dt, ad.y = now["t"].data_ptr(), now["dt"].data_ptr(), now["y"].data_ptr()
        ad.ratio_prev, ad.ratio_pprev = now["prev"].data_ptr(), now["pprev"].data_ptr()
        ad.moved, ad.running_next = moved.data_ptr(), running_next.data_ptr()
        for i in range(7):
            ad.k[i] = ks[i].data_ptr()
        ad.y1 = inputs[6][0].data_ptr()
        names = ("a_y", "a_k0", "a_t", "a_dt", "a_prev", "a_pprev")
        held = [None if adj is None else adj[j] for j in range(6)]
        for name, value in zip(names, held):
            setattr(ad, name, _lib.ptr(value))
        _lib.check(lib.tode_step_finish_backward(aref, cref, stream), "tode_step_finish_backward")
        # ---- the stages reversed: f's vector-Jacobian products by autograd, the sums by the kernel ----
        for i in range(6, 0, -1):
            yi, ti, ki = inputs[i]
            if ki.requires_grad:
                grads = torch.autograd.grad(ki, [yi, ti] + params, g_k[i], allow_unused=True, retain_graph=True)
            else:
                grads = [None] * (2 + len(params))
            g_yi = grads[0] if grads[0] is not None else torch.zeros_like(yi)
            if i == 6:
                g_yi = g_yi + g_y1
            g_ti = None if grads[1] is None else grads[1].to(ttype).contiguous()
            _lib.check(lib.tode_step_stage_backward(aref, cref, i, g_yi.to(dtype).contiguous().data_ptr(), _lib.ptr(g_ti), stream), "tode_step_stage_backward")
            for j, g in enumerate(grads[2:]):
                grad_params[j] = _add(grad_params[j], g)
        adj = (g_y.clone(), g_k[0].clone(), g_t.clone(), g_dt.clone(), g_hist[0].clone(), g_hist[1].clone())

    # the gradients of the times go to the entries of `params` that stand for them
    for given, collected in ((problem_time(replay, "t_start"), g_t_start), (problem_time(replay, "t_end"), g_t_end),
                             (problem_time(replay, "t_eval"), g_t_eval), (dt0 if fixed else None, g_fixed_dt)):
        if collected is None:
            continue
        for j, q in enumerate(params):
            if q is given:
                grad_params[j] = _add(grad_params[j], collected.to(q.dtype))
                break
    out = {k: None for k in STATE_NAMES}
    if adj is not None:
        out = dict(zip(STATE_NAMES, adj))
    return out, grad_params


def problem_time(replay: Replay, name: str):
    return getattr(replay, name)


class SolveThroughLoop(torch.autograd.Function):
    """Forward: the per-step kernels with a record.  Backward: the reverse sweep over it."""

    @staticmethod
    def forward(ctx, adjoint, problem, term, dt0, args, y0, *params):
        record = LoopRecord()
        detached = lambda x: None if x is None else x.detach()
        plain = InitialValueProblem(y0.detach(), detached(problem.t_start), detached(problem.t_end), detached(problem.t_eval))
        with torch.no_grad():
            solution = None
            if getattr(adjoint, "record_in_whole_solve_kernel", True) and adjoint._persistent_ok(plain, term):
                # a built-in term: the forward pass stays in the whole-solve kernels, and the general one writes the record
                solution = adjoint._solve_persistent(plain, term, detached(dt0), record=record)
            if solution is not None:
                pass
            elif adjoint._fused_ok(plain, term):
                solution = adjoint._solve_stepwise(plain, term, detached(dt0), args, record=record)
            else:  # Heun, Euler: the operator path keeps the record
                solution = adjoint._solve_protocol(plain, term, term, detached(dt0), args, record=record)
        ctx.adjoint, ctx.problem, ctx.term, ctx.dt0, ctx.args = adjoint, plain, term, dt0, args
        # the times as the caller gave them: those that require grad are among `params`
        ctx.times = InitialValueProblem(plain.y0, problem.t_start, problem.t_end, problem.t_eval)
        ctx.record, ctx.params = record, params
        ctx.n_initialized = solution.stats["n_initialized"]
        stats = solution.stats
        n_f_evals = stats["n_f_evals"] if "n_f_evals" in stats else torch.empty(0, dtype=torch.long)
        outs = (solution.ys, solution.status, stats["n_steps"], stats["n_accepted"], stats["n_initialized"], n_f_evals)
        ctx.mark_non_differentiable(*outs[1:])
        return outs

    @staticmethod
    def backward(ctx, grad_ys, *unused):
        adjoint, problem, term, params = ctx.adjoint, ctx.problem, ctx.term, list(ctx.params)
        if ctx.record.flags is not None and ctx.record.flags.tolist()[_lib.FLAG_NEEDS_GENERAL]:
            raise RuntimeError("the record of the loop state was too short for the solve it was sized from")
        # (a second initialized point of some sample was written by an iteration: the usual case, told by one reduction)
        some_iteration_wrote = problem.n_evaluation_points > 1 and int(ctx.n_initialized.max()) > 1
        if problem.n_evaluation_points > 0 and not some_iteration_wrote and not ctx.record.any_point_written(problem):
            # No iteration wrote an evaluation point (every sample's points lie at t_start, or the batch stopped before
            # one was reached): ys is a copy of y0 where t_eval[:, 0] == t_start and nothing else, so in the reference's
            # graph no parameter and no time is connected to it: autograd reports them unused, not zero.
            at_start = problem.t_eval[:, 0] == problem.t_start
            first = torch.where(at_start[:, None], grad_ys[:, 0], torch.zeros_like(grad_ys[:, 0]))
            return (None, None, None, None, None, first, *([None] * len(params)))
        # The sweep works on leaves of its own for the times and the tensors in args: one of them may be computed
        # from another (t_start is usually a column of t_eval), and a gradient taken with respect to both would
        # reach the first one twice, once here and once when autograd carries the second one's gradient on.
        stand_in = {}

        def leaf(x):
            if x is None or not x.requires_grad or isinstance(x, torch.nn.Parameter):
                return x
            if id(x) not in stand_in:
                stand_in[id(x)] = x.detach().requires_grad_()
            return stand_in[id(x)]

        times = InitialValueProblem(problem.y0, leaf(ctx.times.t_start), leaf(ctx.times.t_end), leaf(ctx.times.t_eval))
        dt0 = leaf(ctx.dt0)
        args = map_tensors(ctx.args, leaf)
        params = [stand_in.get(id(p), p) for p in params]
        replay = Replay(adjoint.step_method, adjoint.step_size_controller, term, args, times, adjoint.backprop_through_step_size_control, dt0)
        E = problem.n_evaluation_points
        y0 = problem.y0
        add = _add
        F = y0.shape[1]
        use_kernels = getattr(adjoint, "backward_kernels", True) and adjoint._fused_ok(problem, term)
        # one kernel for the whole sweep: a built-in small system whose forward pass wrote its record in the kernel,
        # time and data in one dtype, every gradient asked for within the kernel's reach (state, times, the term's table)
        use_whole = (
            use_kernels
            and getattr(adjoint, "backward_whole_kernel", True)
            and getattr(ctx.record, "arrays", None) is not None
            and problem.time_dtype == problem.data_dtype
            and not term.with_args
        )
        global LAST_SWEEP
        LAST_SWEEP = "whole" if use_whole else ("kernels" if use_kernels else "torch")  # (looked at by the tests)
        swept = reverse_sweep_whole(adjoint, replay, term, problem, dt0, ctx.record, grad_ys, params) if use_whole else None
        if swept is not None:
            adj, grad_params = swept
        else:
            LAST_SWEEP = "kernels" if use_kernels else "torch"
            states = ctx.record.trimmed(ctx.record.iterations)
            hits = simulate_hits(replay, states, E)
            if use_kernels:
                adj, grad_params = reverse_sweep_kernels(adjoint, replay, term, args, problem, ctx.dt0, dt0, states, hits, grad_ys, params, list(ctx.params))
            else:
                adj, grad_params = reverse_sweep_torch(replay, states, hits, grad_ys, params)

        # ---- the start of the loop: y = y0, k0 = f(t_start, y0), dt from the start step rule or dt0 ----
        if adj.get("through_start"):  # (the whole-sweep kernel went through it as well)
            grad_y0 = adj["y"]
        else:
            grad_y0 = SolveThroughLoop.start_backward(ctx, replay, adj, y0, dt0, params, grad_params)
        if E > 0:
            at_start = problem.t_eval[:, 0] == problem.t_start
            first = torch.where(at_start[:, None], grad_ys[:, 0], torch.zeros_like(grad_ys[:, 0]))
            grad_y0 = add(grad_y0, first)
        return (None, None, None, None, None, grad_y0, *grad_params)

    @staticmethod
    def start_backward(ctx, replay, adj, y0, dt0, params, grad_params):
        """The cotangents of the first loop state carried on to ``y0`` (returned) and to ``params`` (added into
        ``grad_params``) by autograd over the start of the loop written as torch operations."""
        add = _add
        with torch.enable_grad():
            y_in = y0.detach().requires_grad_()
            targets, cotangents = [], []
            if adj["y"] is not None:
                targets.append(y_in * 1.0)
                cotangents.append(adj["y"])
            if adj["t"] is not None and replay.t_start.requires_grad:
                targets.append(replay.t_start * 1.0)
                cotangents.append(adj["t"])
            need_f0 = adj["k0"] is not None or (adj["dt"] is not None and ctx.dt0 is None and replay.through_control)
            if need_f0:
                f0 = replay.f(replay.t_start, y_in)
                if adj["k0"] is not None:
                    targets.append(f0)
                    cotangents.append(adj["k0"])
            if adj["dt"] is not None and replay.through_control:
                dt_first = replay.first_step(y_in, f0) if dt0 is None else dt0.to(replay.t_start.dtype)
                # (torch.clamp as in reference adjoints.py:107: on a tie with a bound the step keeps the cotangent)
                dt_first = torch.clamp(dt_first, replay.t_lo - replay.t_start, replay.t_hi - replay.t_start)
                if dt_first.requires_grad:
                    targets.append(dt_first)
                    cotangents.append(adj["dt"])
            grad_y0 = None
            if targets:
                grads = torch.autograd.grad(targets, [y_in] + params, cotangents, allow_unused=True, retain_graph=True)
                grad_y0 = grads[0]
                for i, g in enumerate(grads[1:]):
                    grad_params[i] = add(grad_params[i], g)
        return grad_y0


def solve(adjoint, problem: InitialValueProblem, term, dt0: Optional[torch.Tensor], args: Any):
    """``AutoDiffAdjoint.solve`` for a ``y0``, term parameters or tensors in ``args`` that require grad."""
    from .solution import Solution

    params = [p for p in term.parameters() if p.requires_grad]
    # buffers that require grad (the built-in terms keep their parameters as buffers) and what f closes over, down
    # to the leaves they were computed from; then the tensors handed in by the caller
    for extra in captured_leaves(term, problem, args) + tensor_leaves(args) + [problem.t_start, problem.t_end, problem.t_eval, dt0]:
        if extra is not None and extra.requires_grad and not any(extra is p for p in params):
            params.append(extra)
    ys, status, n_steps, n_accepted, n_initialized, n_f_evals = SolveThroughLoop.apply(adjoint, problem, term, dt0, args, problem.y0, *params)
    stats = {"n_f_evals": n_f_evals} if term.with_stats else {}
    stats.update(n_steps=n_steps, n_accepted=n_accepted, n_initialized=n_initialized)
    ts = problem.t_eval if problem.t_eval is not None else problem.t_end[:, None]
    return Solution(ts=ts, ys=ys, stats=stats, status=status)
