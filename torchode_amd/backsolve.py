"""Gradients by solving the adjoint equation backwards in time (mirrors torchode/adjoints.py:322-681).

The forward solve stores nothing but its outputs.  The backward pass integrates, from each
evaluation point back to the one before it, the state

    [ adjoint of t | y | adjoint of y | adjoint of every parameter of f ]

whose right-hand side is ``f`` itself together with its vector-Jacobian products with the
negated adjoint of ``y``.  Both directions run through ``AutoDiffAdjoint.solve``, i.e. through
the HIP solve loop; the vector-Jacobian products are torch's (``torch.func`` per sample for
``BacksolveAdjoint``, one ``autograd.grad`` on the joined batch for ``JointBacksolveAdjoint``).
"""
from math import prod
from typing import Any, List, Optional, Sequence, Tuple

import torch
import torch.nn as nn

from .adjoints import AutoDiffAdjoint
from .problems import InitialValueProblem
from .solution import Solution
from .terms import ODETerm


def flatten_tensors(*tensors: torch.Tensor) -> Tuple[List[torch.Size], torch.Tensor]:
    """Lay ``[B, ...]`` tensors side by side as one ``[B, sum]`` matrix; also returns the
    per-sample shapes needed to undo it (reference adjoints.py:322-325)."""
    rows = tensors[0].shape[0]
    return [x.shape[1:] for x in tensors], torch.cat([x.reshape(rows, -1) for x in tensors], dim=1)


def unflatten_tensors(shapes: Sequence[torch.Size], flat: torch.Tensor) -> List[torch.Tensor]:
    """Inverse of :func:`flatten_tensors` (reference adjoints.py:328-341)."""
    pieces = flat.split([prod(s) for s in shapes], dim=1)
    return [piece.reshape(flat.shape[0], *shape) for piece, shape in zip(pieces, shapes)]


def _call_f(term: ODETerm, t, y, args):
    return term.f(t, y, args) if term.with_args else term.f(t, y)


class _SolveThenBacksolve(torch.autograd.Function):
    """reference adjoints.py:344-444"""

    @staticmethod
    def forward(ctx, forward_loop, backward_loop, term, augmented_term, y0, t_start, t_end, t_eval, dt0, backward_dt0, args, *params):
        with torch.no_grad():
            solution = forward_loop.solve(InitialValueProblem(y0, t_start, t_end, t_eval), term=term, dt0=dt0, args=args)
        ctx.backward_loop, ctx.augmented_term, ctx.args, ctx.stats = backward_loop, augmented_term, args, solution.stats
        ctx.save_for_backward(t_start, t_end, t_eval, backward_dt0, solution.ys, *params)
        return solution.ts, solution.ys, solution.stats, solution.status

    @staticmethod
    def backward(ctx, grad_ts, grad_ys, grad_stats, grad_status):
        t_start, t_end, t_eval, dt0, ys, *params = ctx.saved_tensors
        loop, term, args = ctx.backward_loop, ctx.augmented_term, ctx.args
        log = ctx.stats.setdefault("backsolve", [])
        B, E, F = ys.shape
        y_cols, adj_cols = slice(1, 1 + F), slice(1 + F, 1 + 2 * F)

        shapes, state = flatten_tensors(
            ys.new_zeros((B, 1)), ys[:, -1], grad_ys[:, -1], *(p.new_zeros((B, *p.shape)) for p in params)
        )

        def back(state, t_from, t_to):
            problem = InitialValueProblem(state, t_start=t_from, t_end=t_to, t_eval=None)
            solution = loop.solve(problem, term=term, dt0=dt0, args=(shapes, args))
            log.append(solution.stats)
            return solution.ys[:, -1]

        with torch.no_grad():
            if t_eval is None:
                state = back(state, t_end, t_start)
            else:
                for e in range(E - 1, 0, -1):
                    state = back(state, t_eval[:, e], t_eval[:, e - 1])
                    # restart from the stored forward value, and pick up the loss gradient there
                    state[:, y_cols] = ys[:, e - 1]
                    state[:, adj_cols] += grad_ys[:, e - 1]

        _, _, grad_y0, *grad_params = unflatten_tensors(shapes, state)
        return (None, None, None, None, grad_y0, None, None, None, None, None, None, *(g.sum(dim=0) for g in grad_params))


class AugmentedDynamicsTerm(ODETerm):
    """Right-hand side of the backward pass of :class:`BacksolveAdjoint` (reference
    adjoints.py:447-494): per sample, ``f`` and the products of the negated adjoint with the
    Jacobians of ``f`` with respect to ``t``, ``y`` and the parameters.  ``args`` is
    ``(shapes, args of f)`` with the shapes :func:`flatten_tensors` returned for the state."""

    def __init__(self, term: ODETerm, vmap_args_dims=None, vmap_randomness: str = "error"):
        super().__init__(self._augmented, with_stats=term.with_stats, with_args=True)
        self.term = term
        self.vmap_args_dims = vmap_args_dims
        self.vmap_randomness = vmap_randomness
        f, with_args = term.f, term.with_args
        module = f if isinstance(f, nn.Module) else None
        names = [] if module is None else [n for n, _ in module.named_parameters()]
        self._param_values = (lambda: ()) if module is None else (lambda: tuple(p for _, p in module.named_parameters()))
        buffers = {} if module is None else dict(module.named_buffers())

        def one_sample(t, y, adj_y, arg):
            def f_of(values, t_, y_):
                call = (t_, y_, arg) if with_args else (t_, y_)
                if module is None:
                    return f(*call)
                return torch.func.functional_call(module, (dict(zip(names, values)), buffers), call)

            dy, pullback = torch.func.vjp(f_of, self._param_values(), t, y)
            d_params, d_t, d_y = pullback(-adj_y)
            return dy, d_t, d_y, d_params

        self.vjp_vf = torch.func.vmap(one_sample, in_dims=(0, 0, 0, vmap_args_dims), randomness=vmap_randomness)

    def _augmented(self, t, state, args):
        shapes, f_args = args
        _, y, adj_y, *_ = unflatten_tensors(shapes, state)
        dy, d_t, d_y, d_params = self.vjp_vf(t, y, adj_y, f_args)
        return flatten_tensors(d_t[:, None], dy, d_y, *d_params)[1]


class BacksolveAdjoint(nn.Module):
    """Same constructor and ``solve`` signature as the reference (adjoints.py:497-539).  Gradients
    flow to ``problem.y0`` and to the parameters of ``term.f``."""

    def __init__(self, term: ODETerm, step_method, step_size_controller, vmap_args_dims=None, vmap_randomness: str = "error"):
        super().__init__()
        self.term = term
        self.augmented_term = AugmentedDynamicsTerm(term, vmap_args_dims=vmap_args_dims, vmap_randomness=vmap_randomness)
        self.forward_adjoint = AutoDiffAdjoint(step_method, step_size_controller)
        self.backward_adjoint = AutoDiffAdjoint(step_method, step_size_controller)

    def solve(self, problem: InitialValueProblem, term: Optional[ODETerm] = None, dt0: Optional[torch.Tensor] = None,
              args: Any = None, backward_dt0: Optional[torch.Tensor] = None) -> Solution:  # fmt: skip
        if backward_dt0 is None and dt0 is not None:
            backward_dt0 = -dt0
        ts, ys, stats, status = _SolveThenBacksolve.apply(
            self.forward_adjoint, self.backward_adjoint, self.term, self.augmented_term, problem.y0, problem.t_start,
            problem.t_end, problem.t_eval, dt0, backward_dt0, args, *self.term.parameters(),
        )  # fmt: skip
        return Solution(ts, ys, stats, status)

    def __repr__(self):
        return (
            f"BacksolveAdjoint(term={self.term!r}, augmented_term={self.augmented_term!r}, "
            f"forward_adjoint={self.forward_adjoint!r}, backward_adjoint={self.backward_adjoint!r})"
        )


class UnwrappingODETerm(ODETerm):
    """The whole batch as ONE sample of ``B * F`` features on the time axis of sample 0 (reference
    adjoints.py:542-569).  ``args`` is ``(B, t_intercept, t_slope, args of f)``: sample ``b``'s own
    time is ``t_intercept[b] + t_slope[b] * t``, and its derivative picks up the factor
    ``t_slope[b]`` by the substitution rule."""

    def __init__(self, term: ODETerm):
        super().__init__(self._joined, with_stats=term.with_stats, with_args=True)
        self.term = term

    def _joined(self, t, y, args):
        batch, t_intercept, t_slope, f_args = args
        own_t = torch.addcmul(t_intercept, t_slope, t)
        dy = _call_f(self.term, own_t, y[0].reshape(batch, -1), f_args)
        return (dy * t_slope[:, None]).reshape(1, -1)


class JointAugmentedDynamicsTerm(ODETerm):
    """Backward right-hand side of :class:`JointBacksolveAdjoint` (reference adjoints.py:572-612):
    one reverse-mode sweep through ``f`` on the joined batch."""

    def __init__(self, term: UnwrappingODETerm):
        super().__init__(self._augmented, with_stats=term.with_stats, with_args=True)
        self.term = term
        self._params = list(term.parameters())

    def _augmented(self, t, state, args):
        shapes, joined_args = args
        _, y, adj_y, *_ = unflatten_tensors(shapes, state)
        with torch.enable_grad():
            t_in, y_in = t.detach().requires_grad_(), y.detach().requires_grad_()
            dy = _call_f(self.term, t_in, y_in, joined_args)
            d_t, d_y, *d_params = torch.autograd.grad(dy, [t_in, y_in, *self._params], -adj_y, allow_unused=True)
        zero_if_unused = lambda g, like: torch.zeros_like(like) if g is None else g
        d_t, d_y = zero_if_unused(d_t, t), zero_if_unused(d_y, y)
        d_params = [zero_if_unused(g, p)[None] for g, p in zip(d_params, self._params)]
        return flatten_tensors(d_t[:, None], dy.detach().reshape(1, -1), d_y, *d_params)[1]


class JointBacksolveAdjoint(nn.Module):
    """Solves the batch as one joined sample, so that one adjoint state (and one set of parameter
    adjoints) serves all of it; every sample must be evaluated at the same relative points of its
    interval (reference adjoints.py:615-681)."""

    def __init__(self, term: ODETerm, step_method, step_size_controller):
        super().__init__()
        self.term = UnwrappingODETerm(term)
        self.augmented_term = JointAugmentedDynamicsTerm(self.term)
        self.forward_loop = AutoDiffAdjoint(step_method, step_size_controller)
        self.backward_loop = AutoDiffAdjoint(step_method, step_size_controller)

    def solve(self, problem: InitialValueProblem, term: Optional[ODETerm] = None, dt0: Optional[torch.Tensor] = None,
              args: Any = None, backward_dt0: Optional[torch.Tensor] = None) -> Solution:  # fmt: skip
        t_eval = problem.t_eval
        if t_eval is not None:
            gaps = torch.diff(t_eval, dim=1)
            relative = gaps / torch.maximum(gaps[:, :1], t_eval.new_tensor(1e-8))
            assert (relative - relative[0]).abs().max() < 1e-8, (
                "JointBacksolveAdjoint can only be applied if all instances in the batch are evaluated at the same "
                "points in time"
            )
            t_eval = t_eval[:1]
        # the affine map from sample 0's interval onto each sample's own
        length = problem.t_end - problem.t_start
        t_slope = length / length[0]
        t_intercept = problem.t_start - t_slope * problem.t_start[0]

        if backward_dt0 is None and dt0 is not None:
            backward_dt0 = -dt0
        _, ys, stats, status = _SolveThenBacksolve.apply(
            self.forward_loop, self.backward_loop, self.term, self.augmented_term, problem.y0.reshape(1, -1),
            problem.t_start[:1], problem.t_end[:1], t_eval, dt0, backward_dt0,
            (problem.batch_size, t_intercept, t_slope, args), *self.term.parameters(),
        )  # fmt: skip
        ys = ys[0].unflatten(1, (problem.batch_size, -1)).transpose(0, 1)
        return Solution(problem.t_end if problem.t_eval is None else problem.t_eval, ys, stats, status)

    def __repr__(self):
        return (
            f"JointBacksolveAdjoint(term={self.term!r}, augmented_term={self.augmented_term!r}, "
            f"forward_loop={self.forward_loop!r}, backward_loop={self.backward_loop!r})"
        )
