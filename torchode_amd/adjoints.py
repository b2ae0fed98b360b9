"""The solve driver (mirrors torchode/adjoints.py:26-319)."""
from functools import partial
from typing import Any, Dict, Optional

import torch
import torch.nn as nn

from . import _lib, differentiable
from .builtin_terms import BuiltinTerm
from .problems import InitialValueProblem
from .interpolation import _PolynomialInterpolation
from .single_step_methods import Dopri5, Euler, Heun, Tsit5
from .solution import Solution
from .step_size_controllers import FixedStepController, IntegralController, PIDController
from .terms import ODETerm

_PROTOCOL_NAMES = (
    "init", "step", "merge_states", "build_interpolation", "convergence_order", "adapt_step_size", "update_state",
    "initial_state", "dt_factor", "_select_initial_step",
)  # fmt: skip


_F_EVAL_VALUES: Dict[int, torch.Tensor] = {}  # count -> 0-dim int64 tensor (never written to)


def _f_evals(count: int, batch: int) -> torch.Tensor:
    """``stats["n_f_evals"]``: int64 ``[B]`` on the CPU, every sample carrying the same count (the
    reference counts evaluations of ``f`` on the whole batch, terms.py:41-63).  One stored value
    viewed ``B`` times: filling half a megabyte per solve costs more than the kernel launch."""
    value = _F_EVAL_VALUES.get(count)
    if value is None:
        if len(_F_EVAL_VALUES) > 4096:
            _F_EVAL_VALUES.clear()
        value = _F_EVAL_VALUES[count] = torch.tensor(count, dtype=torch.long)
    return value.expand(batch)


_PROTOCOL_NAME_SET = frozenset(_PROTOCOL_NAMES)


def _library_object(obj, classes) -> bool:
    """True if ``obj`` is exactly one of the library's classes with no protocol method replaced on
    the instance; only then may a fused kernel stand in for the calls the loop would make."""
    if type(obj) not in classes:
        return False
    if torch.compiler.is_compiling():  # (spelled so that a tracing compiler can follow it)
        return all(name not in obj.__dict__ for name in _PROTOCOL_NAMES)
    return _PROTOCOL_NAME_SET.isdisjoint(vars(obj))


def _sub(module, name):
    """``module.name`` for an attribute that usually is a submodule: ``nn.Module`` keeps those in a dict of their own and
    finds them only through ``__getattr__``, several times the cost of this lookup on a path that runs per solve."""
    found = module.__dict__.get(name)
    if found is None and not torch.compiler.is_compiling():
        found = module._modules.get(name)
    return getattr(module, name) if found is None else found


def _library_plugins(adjoint, term, methods) -> bool:
    """The part of ``AutoDiffAdjoint._library_setup`` that looks at the plug-in objects only."""
    m, c = _sub(adjoint, "step_method"), _sub(adjoint, "step_size_controller")
    return (
        _library_object(m, methods)
        and _library_object(c, (IntegralController, PIDController, FixedStepController))
        and c.fusable
        and isinstance(term, ODETerm)  # subclasses that only supply f (the backsolve terms) included
        and type(term).vf is ODETerm.vf
        and type(term).init is ODETerm.init
        and "vf" not in term.__dict__
        and "init" not in term.__dict__
    )


class Adjoint:
    """What every adjoint offers (reference adjoints.py:15-23)."""

    def solve(self, problem: InitialValueProblem, term: Optional[ODETerm] = None, dt0: Optional[torch.Tensor] = None, args: Any = None) -> Solution:
        raise NotImplementedError()


def __getattr__(name):
    # the reference keeps its backsolve adjoints in this module; here they have one of their own, which imports this one
    if name in ("BacksolveAdjoint", "JointBacksolveAdjoint"):
        from . import backsolve

        return getattr(backsolve, name)
    raise AttributeError(f"module {__name__!r} has no attribute {name!r}")


class AutoDiffAdjoint(nn.Module):
    """Solves a batch of initial value problems with per-sample adaptive steps.

    Same constructor and ``solve`` signature as the reference.  The solve runs in HIP kernels.
    When ``y0``, a parameter of the term, a tensor in ``args`` or one of the times requires grad it
    takes the per-step kernels (Heun, Euler with gradients: the operator path) and records the loop state per iteration, and the result is
    differentiable (``torchode_amd/autodiff.py``; ``backprop_through_step_size_control`` as in the
    reference).
    """

    def __init__(
        self,
        step_method,
        step_size_controller,
        *,
        max_steps: Optional[int] = None,
        backprop_through_step_size_control: bool = True,
        graph_iterations: Optional[int] = None,
    ):
        super().__init__()
        self.step_method = step_method
        self.step_size_controller = step_size_controller
        self.max_steps = max_steps
        self.backprop_through_step_size_control = backprop_through_step_size_control
        # Not in the reference (its counterpart is compiling the loop, docs/jit.ipynb): with a user's
        # torch right-hand side the loop is bound by kernel launches, about 60 per iteration.  With
        # graph_iterations = n, a solve runs its first iterations as usual, then records n iterations
        # (the per-step kernels and whatever f launches) into a HIP graph once and replays it until
        # the batch has stopped.  Only for an f that is safe to record: same kernels for any input
        # values, no host synchronisation, no Python side effects it relies on (f is not called
        # again during replays).
        self.graph_iterations = graph_iterations
        # Set to False to route built-in terms through the general whole-solve kernel only
        # (same results; used by the tests to compare the two kernels).
        self.use_fast_path = True
        # torch.ops.torchode_amd.*: registered here, where no tracer is looking, so that torch.compile of `solve`
        # finds the operators and their tracing rules in place
        from . import ops

        ops.load()

    # ------------------------------------------------------------------ #
    def solve(
        self,
        problem: InitialValueProblem,
        term: Optional[ODETerm] = None,
        dt0: Optional[torch.Tensor] = None,
        args: Any = None,
    ) -> Solution:
        if torch.compiler.is_compiling():
            # Under a tracing compiler (torch.compile of this method): a whole solve with a built-in term is one
            # operator of PyTorch's dispatcher; every other solve leaves the captured program and runs as it does eagerly.
            return self._solve_traced(problem, term, dt0, args)
        return self._solve_eager(problem, term, dt0, args)

    def _solve_traced(self, problem: InitialValueProblem, term: Optional[ODETerm], dt0, args) -> Solution:
        from . import ops

        term_ = term if term is not None else getattr(self.step_method, "term", None)
        f = getattr(term_, "f", None)
        tensors = [problem.y0, problem.t_start, problem.t_end, problem.t_eval, dt0]
        if (
            term_ is None
            or not isinstance(f, BuiltinTerm)
            or not self._persistent_ok(problem, term_)
            or not problem.y0.is_cuda
            or (torch.is_grad_enabled() and any(x is not None and x.requires_grad for x in [*tensors, *f.buffers(), *f.parameters()]))
            or not self._whole_solve_shape(problem, f)
        ):
            return self._solve_eager_outside_the_trace(problem, term, dt0, args)
        kind, control = self.step_size_controller.control_values()
        dtype, B, E = problem.data_dtype, problem.batch_size, problem.n_evaluation_points
        mlp = f.builtin_kind == _lib.TERM_MLP
        params = None if mlp else f.builtin_params().to(dtype)
        shared = ops.mlp_pack_weights(f.builtin_shared().to(dtype), _lib.MLP_INPUTS[f.matrix_inputs], problem.n_features) if mlp else None
        scalars = [float(x) for x in getattr(f, "builtin_scalars", lambda: ())()]
        ys, n_steps, n_accepted, n_initialized, status, iterations = ops.solve_builtin(
            problem.y0, problem.t_start, problem.t_end, problem.t_eval, dt0, params, shared, self.step_method.method_id, f.builtin_kind,
            scalars, kind, control, self.max_steps, self.use_fast_path,
        )  # fmt: skip
        stats: Dict[str, Any] = {}
        if term_.with_stats:
            stats["n_f_evals"] = ((2 if dt0 is None else 1) + 6 * iterations).expand(B)
        stats["n_steps"], stats["n_accepted"], stats["n_initialized"] = n_steps, n_accepted, n_initialized
        ts = problem.t_eval if problem.t_eval is not None else problem.t_end[:, None]
        return Solution(ts=ts, ys=ys, stats=stats, status=status)

    def _whole_solve_shape(self, problem: InitialValueProblem, f: BuiltinTerm) -> bool:
        """What can be told from shapes and settings alone about whether a whole-solve kernel takes the problem (the
        library decides for good, tode_solve_builtin_auto; the eager path asks it and goes on to the per-step kernels on
        a refusal, a captured program cannot)."""
        if f.builtin_kind in _lib.GENERAL_TERMS:
            return True
        c, E, F = self.step_size_controller, problem.n_evaluation_points, problem.n_features
        if c.dt_min is not None or c.dt_max is not None or problem.data_dtype != problem.time_dtype:
            return False
        if f.builtin_kind == _lib.TERM_REACTION_DIFFUSION:
            return (F in (16 * 16, 32 * 32, 64 * 64) and E <= 8192) or (F == 128 * 128 and problem.data_dtype == torch.float32 and E <= 4096)
        return problem.data_dtype == torch.float32 and 1 <= F <= 64 and f.W1.shape[1] == F + 1 and 1 <= f.W1.shape[0] <= 256 and E <= 512

    @torch.compiler.disable
    def _solve_eager_outside_the_trace(self, problem, term, dt0, args) -> Solution:
        return self._solve_eager(problem, term, dt0, args)

    def _solve_eager(self, problem: InitialValueProblem, term: Optional[ODETerm], dt0, args) -> Solution:
        term_ = term if term is not None else getattr(_sub(self, "step_method"), "term", None)
        assert term_ is not None, "no ODE term given, neither to solve() nor to the step method"
        _lib.require_device(problem.y0, problem.t_start, problem.t_end, problem.t_eval, dt0)
        grad_on = torch.is_grad_enabled()
        wants_grad = grad_on and (
            problem.y0.requires_grad
            or problem.t_start.requires_grad
            or problem.t_end.requires_grad
            or (problem.t_eval is not None and problem.t_eval.requires_grad)
            or (dt0 is not None and dt0.requires_grad)
        )
        if grad_on and not wants_grad:
            # a parameter or buffer of the term (the built-in terms keep mu, rho, k, D, the weights as buffers), a
            # tensor in args, or one that f closes over: the reference's loop of torch operations carries gradients
            # to all of them, so no kernel path that returns a result without a graph may take such a solve
            from .autodiff import wants_grad_through_term

            # (f is evaluated once to look for captured tensors, and only where the library's own step methods
            # would call it: a user-defined method may never evaluate f at all)
            wants_grad = wants_grad_through_term(term_, problem, args, probe=False)
            if not wants_grad and not isinstance(getattr(term_, "f", None), BuiltinTerm) and self._library_setup(problem, term_, (Dopri5, Tsit5, Heun, Euler)):
                wants_grad = wants_grad_through_term(term_, problem, args, probe=True)
        if not wants_grad and self._persistent_ok(problem, term_):
            sol = self._solve_persistent(problem, term_, dt0)
            if sol is not None:
                return sol
        if wants_grad and self._library_setup(problem, term_, (Dopri5, Tsit5, Heun, Euler)):
            # gradients through the loop with the library's own plug-ins: forward in the per-step kernels (Dopri5,
            # Tsit5) or on the operator path (Heun, Euler) with a record of the loop state, backward by a reverse
            # sweep over the record
            from . import autodiff

            return autodiff.solve(self, problem, term_, dt0, args)
        # (with a user-defined plug-in a solve that wants gradients takes the operator path below like any other:
        # its kernels' results carry graph nodes wherever an input requires grad, torchode_amd/differentiable.py)
        if self._stepwise_ok(problem, term_):
            return self._solve_stepwise(problem, term_, dt0, args)
        return self._solve_protocol(problem, term, term_, dt0, args)

    # ------------------------------------------------------------------ #
    def _fused_ok(self, problem: InitialValueProblem, term: ODETerm) -> bool:
        return self._library_setup(problem, term, (Dopri5, Tsit5))

    def _library_setup(self, problem: InitialValueProblem, term: ODETerm, methods) -> bool:
        """One of ``methods`` and a controller as the library ships them (no overridden protocol method, the RMS
        norm), a plain term, float32 / float64 tensors."""
        return _library_plugins(self, term, methods) and problem.data_dtype in _lib.DTYPES and problem.time_dtype in _lib.DTYPES

    def _persistent_ok(self, problem: InitialValueProblem, term: ODETerm) -> bool:
        f = _sub(term, "f")
        return (
            isinstance(f, BuiltinTerm)
            and self._fused_ok(problem, term)
            # (time and data in different dtypes: the general kernel of the three small systems is built for them)
            and (problem.data_dtype == problem.time_dtype or f.builtin_kind in _lib.GENERAL_TERMS)
            and type(_sub(self, "step_size_controller")) is not FixedStepController
            and f.builtin_kind in _lib.PERSISTENT_TERMS
            and not term.with_args
        )

    def _stepwise_ok(self, problem: InitialValueProblem, term: ODETerm) -> bool:
        return self._library_setup(problem, term, (Dopri5, Tsit5, Heun, Euler))

    # ------------------------------------------------------------------ #
    def _solve_protocol(self, problem: InitialValueProblem, term: Optional[ODETerm], term_: ODETerm, dt0, args, record=None) -> Solution:
        """The loop of the reference (adjoints.py:50-311) against the plug-in protocols: any step
        method, controller and interpolant, the library's or the user's.  The protocol methods are
        called in the reference's order with the reference's arguments; the bookkeeping between them
        is one kernel per iteration, and the host reads one small flag block per iteration (the
        reference synchronises there as well)."""
        lib = _lib.load()
        method, controller = self.step_method, self.step_size_controller
        dev, dtype, ttype = problem.device, problem.data_dtype, problem.time_dtype
        code = _lib.dtype_code(dtype, ttype)  # time and data may differ (float32 / float64 each)
        B, F, E = problem.batch_size, problem.n_features, problem.n_evaluation_points
        stream = _lib.stream_of(problem.y0)
        t_start, t_end = problem.t_start.contiguous(), problem.t_end.contiguous()
        t_eval = None if problem.t_eval is None else problem.t_eval.contiguous()
        y = problem.y0.contiguous()
        t = t_start
        new = lambda *shape, dt=dtype: torch.empty(shape, dtype=dt, device=dev)

        def as_float(x, shape, to=dtype):
            x = torch.as_tensor(x, device=dev)
            return x.to(to).expand(shape).contiguous()

        def as_status(x):
            return None if x is None else torch.as_tensor(x, device=dev).to(torch.long).expand((B,)).contiguous()

        stats: Dict[str, Any] = {}
        term_.init(problem, stats)
        order = method.convergence_order()
        dt, controller_state, f0 = controller.init(term, problem, order, dt0, stats=stats, args=args)
        method_state = method.init(term, problem, f0, stats=stats, args=args)

        ys = new(B, max(E, 1), F)
        pending = new(B, E, dt=torch.uint8) if E > 0 else None
        dt_in = as_float(dt, (B,), ttype)

        def begin_kernel():
            dt = new(B, dt=ttype)
            rc = lib.tode_loop_begin(
                code, B, F, E, _lib.ptr(t_start), _lib.ptr(t_end), _lib.ptr(t_eval), _lib.ptr(y), _lib.ptr(dt_in), _lib.ptr(dt),
                _lib.ptr(pending), _lib.ptr(ys), stream,
            )  # fmt: skip
            _lib.check(rc, "tode_loop_begin")
            return dt

        # Where an input requires grad, every kernel's result carries a graph node that differentiates the same
        # operation written as torch operations (differentiable.through), so the solve is differentiable for any mix of
        # the library's and a user's plug-ins, as the reference's loop of torch operations is (adjoints.py:135-260).
        dt = differentiable.through(begin_kernel, differentiable.loop_begin, t_start, t_end, dt_in)
        if E > 0 and differentiable.tracked(y):
            at_start = (t_eval[:, 0] == t_start).nonzero()[:, 0]
            ys[at_start, 0] = y[at_start]  # (the kernel wrote the same values; this write is the one autograd sees)
        if not self.backprop_through_step_size_control:
            dt = dt.detach()

        running = torch.ones(B, dtype=torch.bool, device=dev)
        n_steps = torch.zeros(B, dtype=torch.long, device=dev)
        n_accepted = torch.zeros(B, dtype=torch.long, device=dev)
        flags = new(_lib.LOOP_FLAG_WORDS, dt=torch.int32)

        a = _lib.LoopArgs()
        a.dtype, a.n_features, a.n_eval, a.batch = code, F, E, B
        a.max_steps = -1 if self.max_steps is None else int(self.max_steps)
        a.t_start, a.t_end = t_start.data_ptr(), t_end.data_ptr()
        a.t_eval = None if t_eval is None else t_eval.data_ptr()
        a.n_steps, a.n_accepted = n_steps.data_ptr(), n_accepted.data_ptr()
        a.pending = None if pending is None else pending.data_ptr()
        a.flags = flags.data_ptr()

        while True:
            if record is not None:
                record.snapshot_protocol(t, dt, y, controller_state, running, n_accepted)
            step_result, interp_data, method_state_next, method_status = method.step(
                term, running, y, t, dt, method_state, stats=stats, args=args
            )
            accept, dt_next, controller_state_next, controller_status = controller.adapt_step_size(
                t, dt, y, step_result, controller_state, stats
            )

            if not self.backprop_through_step_size_control:
                dt_next = dt_next.detach() if isinstance(dt_next, torch.Tensor) else dt_next

            # ---- one kernel: state update, counters, running, status, evaluation mask, next dt ----
            y_new = as_float(step_result.y, (B, F))
            accept_ = torch.as_tensor(accept, device=dev).to(torch.bool).expand((B,)).contiguous()
            dt_next_ = as_float(dt_next, (B,), ttype)
            m_status, c_status = as_status(method_status), as_status(controller_status)
            running_out, to_update = new(B, dt=torch.bool), new(B, dt=torch.bool)
            status = new(B, dt=torch.long)
            to_evaluate = new(B, E, dt=torch.uint8) if E > 0 else None

            def advance_kernel(t=t, dt=dt, y=y, y_new=y_new, dt_next_=dt_next_):
                t_out, dt_out, y_out = new(B, dt=ttype), new(B, dt=ttype), new(B, F)
                a.t, a.dt, a.y, a.running = t.data_ptr(), dt.data_ptr(), y.data_ptr(), running.data_ptr()
                a.y_new, a.accept, a.dt_next = y_new.data_ptr(), accept_.data_ptr(), dt_next_.data_ptr()
                a.method_status = None if m_status is None else m_status.data_ptr()
                a.controller_status = None if c_status is None else c_status.data_ptr()
                a.t_out, a.dt_out, a.y_out = t_out.data_ptr(), dt_out.data_ptr(), y_out.data_ptr()
                a.running_out, a.to_update, a.status = running_out.data_ptr(), to_update.data_ptr(), status.data_ptr()
                a.to_evaluate = None if to_evaluate is None else to_evaluate.data_ptr()
                _lib.check(lib.tode_loop_advance(_lib.C.byref(a), stream), "tode_loop_advance")
                return t_out, dt_out, y_out

            t_out, dt_out, y_out = differentiable.through(
                advance_kernel, partial(differentiable.loop_advance, to_update, running_out), t_start, t_end, t, dt, y, y_new, dt_next_
            )
            fl = flags.tolist()  # the iteration's host synchronisation

            method_state = method.merge_states(to_update, method_state_next, method_state)

            # ---- dense output at the evaluation points this step passed ----
            if E > 0 and fl[_lib.LOOP_N_TO_EVALUATE] > 0:
                interpolation = method.build_interpolation(interp_data)
                own = isinstance(interpolation, _PolynomialInterpolation) and type(interpolation).evaluate is _PolynomialInterpolation.evaluate
                if own and not interpolation.tracked(t_eval):
                    interpolation.evaluate_masked(t_eval, to_evaluate, ys)
                else:
                    hit = to_evaluate.view(torch.bool).nonzero()
                    sample_idx, eval_idx = hit[:, 0], hit[:, 1]
                    ys[sample_idx, eval_idx] = interpolation.evaluate(t_eval[sample_idx, eval_idx], sample_idx).to(dtype)

            controller_state = controller.merge_states(running_out, controller_state_next, controller_state)
            t, dt, y, running = t_out, dt_out, y_out, running_out

            if fl[_lib.LOOP_ANY_RUNNING] and not fl[_lib.LOOP_ANY_FAILURE]:
                continue

            if record is not None:
                record.snapshot_protocol(t, dt, y, controller_state, running, n_accepted)
                record.iterations = len(record.states) - 1
            if m_status is None and c_status is None and self.max_steps is None:
                status = torch.tensor(0, dtype=torch.long, device=dev).expand(B)
            stats["n_steps"], stats["n_accepted"] = n_steps, n_accepted
            if E > 0:
                n_init = new(B, dt=torch.long)
                _lib.check(lib.tode_count_initialized(B, E, _lib.ptr(pending), _lib.ptr(n_init), stream), "tode_count_initialized")
                stats["n_initialized"] = n_init
                return Solution(ts=problem.t_eval, ys=ys, stats=stats, status=status)
            interpolation = method.build_interpolation(interp_data)
            y_end = interpolation.evaluate(problem.t_end, torch.arange(B, device=dev))
            stats["n_initialized"] = torch.ones(B, dtype=torch.long, device=dev)
            return Solution(ts=problem.t_end[:, None], ys=y_end[:, None], stats=stats, status=status)

    # Graph replay: how many loop iterations are enqueued between two synchronising looks at the
    # device flags.  Eager iterations: how many iterations the host may be ahead of the device.
    poll_first, poll_max, run_ahead = 4, 32, 2

    def _solve_stepwise(self, problem: InitialValueProblem, term: ODETerm, dt0, args, record=None) -> Solution:
        """Arbitrary Python ``f``: per-step kernels around the user's torch RHS, loop state on the
        device, no host synchronisation per step (the host polls a flag every few iterations)."""
        lib = _lib.load()
        y0 = problem.y0.contiguous()
        dev, dtype, ttype = y0.device, y0.dtype, problem.time_dtype  # (time and data may differ, problems.py:44-56)
        B, F = y0.shape
        E = problem.n_evaluation_points
        t_start, t_end = problem.t_start.contiguous(), problem.t_end.contiguous()
        t_eval = None if problem.t_eval is None else problem.t_eval.contiguous()
        dt0_ = None if dt0 is None else dt0.to(ttype).contiguous()
        fixed = type(self.step_size_controller) is FixedStepController
        assert not fixed or dt0_ is not None, "Fixed step size solving requires you to configure dt0"
        ctrl = self.step_size_controller.c_struct()
        stream = _lib.stream_of(y0)
        new = lambda *shape, dt=dtype: torch.empty(shape, dtype=dt, device=dev)

        ys = new(B, max(E, 1), F)
        t, dt = new(B, dt=ttype), new(B, dt=ttype)
        y, k0 = new(B, F), new(B, F)
        hist = new(2, B)
        ints = new(6, B, dt=torch.int32)
        pending = new(B, max(E, 1), dt=torch.uint8)
        flags = new(_lib.STEP_FLAG_WORDS, dt=torch.int32)

        s = _lib.StepState()
        s.dtype, s.time_dtype, s.method, s.n_features, s.n_eval = _lib.DTYPES[dtype], _lib.DTYPES[ttype], self.step_method.method_id, F, E
        s.batch = B
        s.max_steps = -1 if self.max_steps is None else int(self.max_steps)
        s.y0, s.t_start, s.t_end = y0.data_ptr(), t_start.data_ptr(), t_end.data_ptr()
        s.t_eval = None if t_eval is None else t_eval.data_ptr()
        s.t, s.dt, s.y, s.k0 = t.data_ptr(), dt.data_ptr(), y.data_ptr(), k0.data_ptr()
        s.ratio_prev, s.ratio_pprev = hist[0].data_ptr(), hist[1].data_ptr()
        s.running, s.cursor, s.n_steps, s.n_accepted, s.status, s.monotone = (ints[i].data_ptr() for i in range(6))
        s.pending, s.ys, s.flags = pending.data_ptr(), ys.data_ptr(), flags.data_ptr()
        # two words in pinned host memory that the device keeps up to date: the host sees the loop end
        # by reading its own memory, after every iteration and without a synchronisation
        mirror = torch.empty(2, dtype=torch.int32, pin_memory=True)
        s.host_flags = mirror.data_ptr()
        s.fixed_dt = dt0_.data_ptr() if fixed else None
        stopped_on_device = mirror.numpy()
        stopped_on_device[:] = 0  # (on the host: torch.zeros on pinned memory costs 0.2 ms)
        sref, cref = _lib.C.byref(s), _lib.C.byref(ctrl)

        f, with_args = term.f, term.with_args

        def rhs(tt, yy):
            out = f(tt, yy, args) if with_args else f(tt, yy)
            if out.dtype != dtype or not out.is_contiguous() or out.shape != yy.shape:
                out = out.to(dtype).expand(yy.shape).contiguous()
            return out

        # Every evaluation of f gets freshly allocated (t, y) tensors, as in the reference, so a
        # caller that keeps them (e.g. to log the evaluation times) sees what f saw.  `keep`
        # holds the buffers of the current iteration alive while kernels still read them.
        keep = {}

        def stage_buffers(i):
            keep["y", i], keep["t", i] = new(B, F), new(B, dt=ttype)
            s.ystage[i], s.tnode = keep["y", i].data_ptr(), keep["t", i].data_ptr()
            return keep["t", i], keep["y", i]

        def evaluate(i, tt, yy):
            keep["k", i] = rhs(tt, yy)
            s.k[i] = keep["k", i].data_ptr()

        # Dopri5 and Tsit5 carry the last stage's derivative into the next step, so f(t_start, y0) is needed before
        # the loop whatever sets the first step; Heun and Euler evaluate their first stage anew in every step
        # (runge_kutta.py:196-212) and see f before the loop only through the controller's start step rule.
        n_stages = {_lib.DOPRI5: 7, _lib.TSIT5: 7, _lib.HEUN: 2, _lib.EULER: 1}[s.method]
        carries = n_stages == 7
        n_init_evals = 0
        if carries or dt0_ is None:
            evaluate(0, t_start, y0)
            n_init_evals = 1
        if dt0_ is None:
            tt, yy = stage_buffers(1)
            _lib.check(lib.tode_step_begin(sref, cref, None, 0, stream), "tode_step_begin")
            evaluate(1, tt, yy)
            _lib.check(lib.tode_step_begin(sref, cref, None, 1, stream), "tode_step_begin")
            n_init_evals = 2
        else:
            s.tnode = t.data_ptr()  # unused by this phase, but must be a valid pointer
            _lib.check(lib.tode_step_begin(sref, cref, _lib.ptr(dt0_), 0, stream), "tode_step_begin")
        if carries:
            s.k[0] = k0.data_ptr()  # from here on the first slot is the state's own buffer
        else:
            keep["y1"] = new(B, F)
            s.ystage[6] = keep["y1"].data_ptr()  # the finish kernel forms the step's result there

        def iterate(n, stream):
            for _ in range(n):
                if record is not None:
                    record.snapshot(t, dt, y, k0, hist, ints)
                if not carries:
                    evaluate(0, t.clone(), y.clone())
                for i in range(1, n_stages):
                    tt, yy = stage_buffers(i)
                    _lib.check(lib.tode_step_stage(sref, cref, i, stream), "tode_step_stage")
                    evaluate(i, tt, yy)
                _lib.check(lib.tode_step_finish(sref, cref, stream), "tode_step_finish")

        use_graph = bool(self.graph_iterations) and record is None
        chunk, graph, replays, enqueued, spins = self.poll_first, None, 1, 0, 0
        while True:
            if graph is not None:
                for _ in range(replays):
                    graph.replay()
            elif use_graph or not self.run_ahead:
                iterate(chunk, stream)
                if not use_graph:
                    chunk = min(2 * chunk, self.poll_max)
            else:
                # Eager iterations: the host looks at the device's stop word (in its own memory) after
                # every iteration it has enqueued.  It runs ahead of the device, so a few iterations
                # are still enqueued after the loop has ended there; their kernels do nothing.
                while not stopped_on_device[0]:
                    if enqueued - int(stopped_on_device[1]) < self.run_ahead:
                        iterate(1, stream)
                        enqueued += 1
                        spins = 0
                    else:  # the device is the slower side: let it finish an iteration before enqueuing more
                        spins += 1
                        if spins > 1_000_000:
                            break  # (no news for long: synchronise below and look again)
            fl = flags.tolist()  # host/device synchronisation
            if fl[_lib.STEP_FLAG_STOPPED]:
                break
            if use_graph and graph is None:
                # (the eager iterations above have also warmed up whatever f uses)
                graph = self._record(lambda st: iterate(int(self.graph_iterations), st), y0)
            elif graph is not None:
                replays = min(2 * replays, max(1, self.poll_max // int(self.graph_iterations)))
        y1_buffer = keep.pop("y1", None)  # (kernels enqueued after the stop do nothing, but hold the pointer)
        keep.clear()
        del graph  # frees the memory f's intermediate tensors were recorded with
        if record is not None:
            record.snapshot(t, dt, y, k0, hist, ints)
            record.iterations = fl[_lib.STEP_FLAG_ITERATIONS]

        out = new(4, B, dt=torch.int64)
        _lib.check(lib.tode_step_stats(sref, *(_lib.ptr(out[i]) for i in range(4)), stream), "tode_step_stats")
        stats: Dict[str, Any] = {}
        if term.with_stats:
            n = n_init_evals + (n_stages - 1 if carries else n_stages) * fl[_lib.STEP_FLAG_ITERATIONS]
            stats["n_f_evals"] = _f_evals(n, B)
        stats["n_steps"], stats["n_accepted"], stats["n_initialized"] = out[0], out[1], out[2]
        ts = problem.t_eval if problem.t_eval is not None else problem.t_end[:, None]
        return Solution(ts=ts, ys=ys, stats=stats, status=out[3])

    @staticmethod
    def _record(body, like: torch.Tensor) -> "torch.cuda.CUDAGraph":
        """Records ``body(stream)`` into a HIP graph on a side stream; nothing runs until a replay.
        Kernels after the batch has stopped do nothing, so replaying whole chunks is safe."""
        graph = torch.cuda.CUDAGraph()
        side = torch.cuda.Stream(device=like.device)  # default priority
        side.wait_stream(torch.cuda.current_stream(like.device))
        with torch.cuda.stream(side):
            graph.capture_begin(capture_error_mode="thread_local")
            try:
                body(_lib.stream_of(like))
            finally:
                graph.capture_end()
        torch.cuda.current_stream(like.device).wait_stream(side)
        return graph

    def _solve_persistent(self, problem: InitialValueProblem, term: ODETerm, dt0, record=None) -> Solution:
        """``record``: a ``LoopRecord`` to fill with the loop state of every iteration (the solve then runs the general
        kernel once more, limited to the iterations the first pass took, with a record of that many entries)."""
        lib = _lib.load()
        f: BuiltinTerm = _sub(term, "f")
        if record is not None and f.builtin_kind not in _lib.GENERAL_TERMS:
            return None  # (the record is written for the three small systems: the grid and MLP terms record on the per-step path)
        method_id, controller = _sub(self, "step_method").method_id, _sub(self, "step_size_controller")
        # What depends on the problem's tensors alone is worked out once per problem object and kept on it (checked by
        # identity, since the attributes of a problem may be reassigned, and by the tensors' version counters, since
        # the plan may hold a contiguous copy of one of them that an in-place update of the original would not reach).
        tensors = (problem.y0, problem.t_start, problem.t_end, problem.t_eval)
        versions = tuple(-1 if x is None else x._version for x in tensors)
        plan = getattr(problem, "_launch_plan", None)
        if plan is None or plan[-1] != versions or any(a is not b for a, b in zip(plan[0], tensors)):
            y0 = problem.y0.contiguous()
            # t_start / t_end are usually columns of t_eval: hand them over with their stride
            t_start, t_end = (t if t.stride(0) >= 1 else t.contiguous() for t in (problem.t_start, problem.t_end))
            t_eval = None if problem.t_eval is None else problem.t_eval.contiguous()
            ts = problem.t_eval if problem.t_eval is not None else problem.t_end[:, None]
            plan = (tensors, y0, t_start, t_end, t_eval, ts, y0.device, y0.dtype, y0.shape[0], y0.shape[1], problem.n_evaluation_points,
                    y0.data_ptr(), t_start.data_ptr(), t_end.data_ptr(), t_start.stride(0), t_end.stride(0),
                    None if t_eval is None else t_eval.data_ptr(), {}, versions)  # fmt: skip
            problem._launch_plan = plan
        _, y0, t_start, t_end, t_eval, ts, dev, dtype, B, F, E, y0_ptr, t_start_ptr, t_end_ptr, t_start_stride, t_end_stride, t_eval_ptr, _, _ = plan
        params = f.builtin_params()
        if params.device != dev or params.dtype != dtype:
            params = params.to(device=dev, dtype=dtype)
        if params.numel() == 0 and params.shape[0] != B:  # a term without per-sample parameters
            params = y0.new_empty((B, 0))
        assert params.shape[0] == B, "built-in term parameters do not match the batch size"
        mlp = f.builtin_kind == _lib.TERM_MLP
        if mlp and (
            dtype != torch.float32 or not 1 <= F <= 64 or f.W1.shape[1] != F + 1 or not 1 <= f.W1.shape[0] <= 256
        ):
            return None  # the matrix-core kernel takes up to 64 features and up to 256 hidden units: the caller takes another path
        shared = f.builtin_packed(dev, dtype) if mlp else None
        ttype = t_start.dtype
        dt0_ = None if dt0 is None else dt0.to(ttype).contiguous()

        ys = torch.empty((B, max(E, 1), F), dtype=dtype, device=dev)
        ctrl = controller.c_struct()
        stream = _lib.stream_of(y0)

        # The argument struct is kept with the plan and copied from there while it describes the same call (same problem
        # tensors, parameters, first step, method, term and step limit): only the output pointer changes from solve to solve.
        key = (method_id, f.builtin_kind, self.max_steps, params.data_ptr(), None if dt0_ is None else dt0_.data_ptr(),
               None if shared is None else shared.data_ptr())  # fmt: skip
        held = plan[-2]
        if held.get("key") != key:
            scal = list(getattr(f, "builtin_scalars", lambda: ())()) + [0.0] * 4
            a = _lib.SolveArgs(  # positional, in the order of struct tode_solve_args
                _lib.dtype_code(dtype, ttype), method_id, f.builtin_kind, F, E, params.shape[1], B,
                -1 if self.max_steps is None else int(self.max_steps), -1, (_lib.C.c_double * 4)(*scal[:4]),
                y0_ptr, t_start_ptr, t_end_ptr, t_start_stride, t_end_stride, t_eval_ptr, None if dt0_ is None else dt0_.data_ptr(),
                params.data_ptr() if params.numel() else None,
                None if shared is None else shared.data_ptr(), 0 if shared is None else shared.numel(),
            )  # fmt: skip  (what the general kernel needs besides lives in the workspace)
            held.update(key=key, args=a, workspace_bytes=lib.tode_solve_workspace_bytes(_lib.C.byref(a)), scalars=tuple(scal[:4]),
                        keep=(params, dt0_, shared))  # fmt: skip
        elif held["scalars"] != tuple((list(getattr(f, "builtin_scalars", lambda: ())()) + [0.0] * 4)[:4]):
            held.clear()  # (a scalar of the term was reassigned: describe the call anew)
            return self._solve_persistent(problem, term, dt0, record=record)
        a = _lib.SolveArgs.from_buffer_copy(held["args"])  # (a copy per call: solves of one problem object may overlap in threads)
        a.ys = ys.data_ptr()
        a_ref = _lib.C.byref(a)

        # One call: the one-kernel path where the batch is in its shape, the general kernel where it is not or where
        # the first reported that the batch leaves the common case, the int64 stats as the reference returns them.
        out = torch.empty((4, B), dtype=torch.int64, device=dev)
        o0, row = out.data_ptr(), 8 * B
        if record is not None:
            # Once a recording solve of this solver has told how many iterations such a batch takes: the solve and its
            # record in one kernel, with a record of a few entries more.  A batch that leaves that kernel's case, or
            # takes more iterations than the record holds, goes the long way below.
            solution = self._solve_recording_in_one_kernel(lib, a, ctrl, out, stream, record, dict(
                B=B, E=E, F=F, dtype=dtype, ttype=ttype, dev=dev, ts=ts, ys=ys, has_dt0=dt0 is not None, with_stats=term.with_stats))  # fmt: skip
            if solution is not None:
                return solution
        workspace = torch.empty(held["workspace_bytes"], dtype=torch.uint8, device=dev)
        iterations = _lib.C.c_int64(0)
        rc = lib.tode_solve_builtin_auto(
            a_ref, _lib.C.byref(ctrl), o0, o0 + row, o0 + 2 * row, o0 + 3 * row, workspace.data_ptr(), held["workspace_bytes"],
            1 if self.use_fast_path else 0, stream, _lib.C.byref(iterations),
        )  # fmt: skip  (returns after the solve's one host synchronisation)
        if rc == _lib.E_UNSUPPORTED:
            return None  # no whole-solve kernel for this case: the caller takes the per-step or the operator path
        if rc:
            _lib.check(rc, "tode_solve_builtin_auto")
        stats: Dict[str, Any] = {}
        if term.with_stats:
            stats["n_f_evals"] = _f_evals((2 if dt0 is None else 1) + 6 * iterations.value, B)
        stats["n_steps"], stats["n_accepted"], stats["n_initialized"], status = out.unbind(0)
        if record is not None:
            # The same solve through the general kernel again, stopped where the first pass stopped, writing the
            # state before every iteration: entry i of every array is what the per-step kernels' loop holds there.
            L, n = iterations.value, iterations.value + 1
            new = lambda *shape, dt=dtype: torch.empty(shape, dtype=dt, device=dev)
            fields, rec = self._record_arrays(n, B, F, dtype, ttype, dev)
            again = _lib.SolveArgs.from_buffer_copy(a)
            scratch_ys, y_idle = new(B, max(E, 1), F), new(B, F)
            counters, flags = new(5, B, dt=torch.int32), new(_lib.FLAG_WORDS, dt=torch.int32)
            pending = new(B, max(E, 1), dt=torch.uint8)
            again.ys, again.y_idle, again.pending, again.flags = scratch_ys.data_ptr(), y_idle.data_ptr(), pending.data_ptr(), flags.data_ptr()
            again.n_steps, again.n_accepted, again.n_initialized, again.status_last, again.status_idle = (counters[i].data_ptr() for i in range(5))
            again.iteration_cap = L
            again.record = _lib.C.addressof(rec)
            _lib.check(lib.tode_solve_builtin(_lib.C.byref(again), _lib.C.byref(ctrl), stream), "tode_solve_builtin")
            record.flags = flags  # (looked at when the backward pass starts: no second wait for the GPU here)
            self._remember_record_entries((B, F, E, dtype, f.builtin_kind), n + 4)  # (the next recording solve of a batch like this one tries it in one kernel)
            record.iterations = L
            record.arrays = fields  # (entry-major arrays: what tode_solve_builtin_backward reads)
        return Solution(ts=ts, ys=ys, stats=stats, status=status)

    def _remember_record_entries(self, shape, entries: int) -> None:
        """How many entries the record of a solve of this shape (batch, features, evaluation points, dtype, term) took,
        plus a margin: what the next recording solve of that shape sizes its record from.  A few shapes are kept."""
        held = self.__dict__.setdefault("_record_entries", {})
        if shape not in held and len(held) >= 8:
            held.clear()
        held[shape] = int(entries)

    @staticmethod
    def _record_arrays(n, B, F, dtype, ttype, dev):
        new = lambda *shape, dt=dtype: torch.empty(shape, dtype=dt, device=dev)
        fields = dict(t=new(n, B, dt=ttype), dt=new(n, B, dt=ttype), y=new(n, B, F), k0=new(n, B, F), prev=new(n, B), pprev=new(n, B),
                      running=new(n, B, dt=torch.int32), n_accepted=new(n, B, dt=torch.int32))  # fmt: skip
        return fields, _lib.SolveRecord(n, *(fields[k].data_ptr() for k in ("t", "dt", "y", "k0", "prev", "pprev", "running", "n_accepted")))

    def _solve_recording_in_one_kernel(self, lib, a, ctrl, out, stream, record, q) -> Optional[Solution]:
        """The solve with its record from one launch of a fast kernel (``tode_solve_builtin_fast`` with a record), or
        None where that is not to be had: no earlier recording solve to size the record from, a shape or controller
        setting outside that kernel's case, a batch that leaves it, or a record that came out too short."""
        shape = (q["B"], q["F"], q["E"], q["dtype"], a.term)
        n = getattr(self, "_record_entries", {}).get(shape)
        if n is None or not getattr(self, "record_in_one_kernel", True) or not self.use_fast_path:
            return None
        if q["E"] == 0 or q["dtype"] != q["ttype"] or a.term in (_lib.TERM_REACTION_DIFFUSION, _lib.TERM_MLP):
            return None
        B = q["B"]
        fields, rec = self._record_arrays(n, B, q["F"], q["dtype"], q["ttype"], q["dev"])
        a.record = _lib.C.addressof(rec)
        fl = (_lib.C.c_int32 * _lib.FLAG_WORDS)()
        o0, row = out.data_ptr(), 8 * B
        rc = lib.tode_solve_builtin_fast_sync(_lib.C.byref(a), _lib.C.byref(ctrl), o0, o0 + row, o0 + 2 * row, o0 + 3 * row, stream, fl)
        a.record = None
        if rc == _lib.E_UNSUPPORTED:
            return None
        _lib.check(rc, "tode_solve_builtin_fast_sync")
        if fl[_lib.FLAG_NEEDS_GENERAL]:
            return None
        L = fl[_lib.FLAG_MAX_ITERATIONS]
        record.iterations, record.arrays = L, fields
        self._remember_record_entries(shape, L + 1 + 4)
        stats: Dict[str, Any] = {}
        if q["with_stats"]:
            stats["n_f_evals"] = _f_evals((1 if q["has_dt0"] else 2) + 6 * L, B)
        stats["n_steps"], stats["n_accepted"], stats["n_initialized"], status = out.unbind(0)
        return Solution(ts=q["ts"], ys=q["ys"], stats=stats, status=status)

    def __repr__(self):
        return (
            f"AutoDiffAdjoint(step_method={self.step_method}, "
            f"step_size_controller={self.step_size_controller}, max_steps={self.max_steps}, "
            f"backprop_through_step_size_control={self.backprop_through_step_size_control}"
            + (f", graph_iterations={self.graph_iterations})" if self.graph_iterations else ")")
        )
