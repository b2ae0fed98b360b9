"""BacksolveAdjoint / JointBacksolveAdjoint: gradients from a second solve backwards in time.

The CPU tests pin the host logic (state packing, the augmented right-hand sides, the sweep over
the evaluation intervals) with the ATen-op oracle standing in for the solve loop.  The GPU tests
restate the reference's cases (tests/adjoint_test.py:372-496) on the kernels.  Independent of
both: for ``dy/dt = y A`` the solution is ``y0 expm(A (t - t0))``, so torch's own autograd
through ``matrix_exp`` gives the gradients the adjoint solve has to reproduce.
"""
import pytest
import torch
import torch.nn as nn

import torchode_amd as to
from oracle import torch_loop
from torchode_amd.backsolve import (
    AugmentedDynamicsTerm,
    JointAugmentedDynamicsTerm,
    UnwrappingODETerm,
    flatten_tensors,
    unflatten_tensors,
)

gpu = pytest.mark.gpu

A0 = [[-1.4534, -0.3726, -0.7916], [-1.0553, 0.9511, 0.1316], [-1.8320, -0.7707, -1.0867]]
Y0 = [[0.33, 1.2, -0.4], [0.55, -0.8, 1.23]]
T_EVAL = [[0.0, 1.77, 3.0], [2.0, 3.5, 6.0]]
T_EVAL_ALIGNED = [[0.0, 1.125, 3.0], [2.0, 3.5, 6.0]]


class LinearDynamics(nn.Module):
    def __init__(self, A):
        super().__init__()
        self.register_parameter("A", A)

    def forward(self, t, y):
        return y @ self.A


class ForcedDynamics(nn.Module):
    """Depends on t, y, two parameters and a buffer."""

    def __init__(self):
        super().__init__()
        self.w = nn.Parameter(torch.tensor([[0.3, -0.2], [0.5, 0.1]], dtype=torch.float64))
        self.b = nn.Parameter(torch.tensor([0.1, -0.4], dtype=torch.float64))
        self.register_buffer("freq", torch.tensor(1.7, dtype=torch.float64))

    def forward(self, t, y):
        return torch.tanh(y @ self.w) * torch.sin(self.freq * t)[..., None] + self.b * t[..., None]


def closed_form_loss(y0, A, t_eval):
    dts = t_eval - t_eval[:, :1]
    ys = torch.einsum("bf,befg->beg", y0, torch.matrix_exp(A[None, None] * dts[:, :, None, None]))
    return ys.mean()


def closed_form_gradients(t_eval, device="cpu"):
    y0 = torch.tensor(Y0, dtype=torch.float64, device=device, requires_grad=True)
    A = torch.tensor(A0, dtype=torch.float64, device=device, requires_grad=True)
    closed_form_loss(y0, A, t_eval.to(device)).backward()
    return y0.grad, A.grad


class OracleLoop(nn.Module):
    """The ATen-op restatement of the solve loop behind AutoDiffAdjoint.solve's signature."""

    controller = torch_loop.Controller("pid", atol=1e-9, rtol=1e-9, pcoeff=0.2, icoeff=0.5, dcoeff=0.0)

    def solve(self, problem, term=None, dt0=None, args=None):
        f = (lambda t, y: term.f(t, y, args)) if term.with_args else term.f
        out = torch_loop.solve(f, problem.y0, problem.t_eval, method="tsit5", controller=self.controller, t_start=problem.t_start,
                               t_end=problem.t_end, dt0=dt0)  # fmt: skip
        ts = problem.t_eval if problem.t_eval is not None else problem.t_end[:, None]
        stats = {k: out[k] for k in ("n_f_evals", "n_steps", "n_accepted", "n_initialized")}
        return to.Solution(ts=ts, ys=out["ys"], stats=stats, status=out["status"])


# ---------------------------------------------------------------------------------------------
# host logic (CPU)
# ---------------------------------------------------------------------------------------------


def test_state_packing_round_trip():
    parts = [torch.randn(4, 1), torch.randn(4, 3), torch.randn(4, 2, 5), torch.randn(4, 0), torch.randn(4, 2, 1, 3)]
    shapes, flat = flatten_tensors(*parts)
    assert flat.shape == (4, 1 + 3 + 10 + 0 + 6) and [tuple(s) for s in shapes] == [(1,), (3,), (2, 5), (0,), (2, 1, 3)]
    assert torch.equal(flat[:, 4:14], parts[2].reshape(4, 10))
    back = unflatten_tensors(shapes, flat)
    assert all(torch.equal(a, b) for a, b in zip(parts, back))


def per_sample_vjps(f, params, t, y, adj):
    """Row b: (f, -adj_b . df/dt, -adj_b . df/dy, -adj_b . df/dparams) of sample b alone."""
    rows = []
    for b in range(y.shape[0]):
        tb, yb = t[b : b + 1].clone().requires_grad_(), y[b : b + 1].clone().requires_grad_()
        dy = f(tb, yb)
        grads = torch.autograd.grad(dy, [tb, yb, *params], -adj[b : b + 1], allow_unused=True)
        grads = [torch.zeros_like(x) if g is None else g for g, x in zip(grads, [tb, yb, *params])]
        rows.append(torch.cat([grads[0], dy.detach()[0], grads[1][0], *(g.reshape(-1) for g in grads[2:])]))
    return torch.stack(rows)


def test_augmented_right_hand_side_is_the_per_sample_vjp():
    torch.manual_seed(0)
    f = ForcedDynamics()
    term = AugmentedDynamicsTerm(to.ODETerm(f))
    B = 5
    t, y, adj = (torch.randn(B, dtype=torch.float64), torch.randn(B, 2, dtype=torch.float64), torch.randn(B, 2, dtype=torch.float64))
    shapes, state = flatten_tensors(torch.zeros(B, 1, dtype=torch.float64), y, adj, torch.zeros(B, 2, 2, dtype=torch.float64),
                                    torch.zeros(B, 2, dtype=torch.float64))  # fmt: skip
    with torch.no_grad():  # the solve loop calls it without grad mode
        out = term.vf(t, state, {"n_f_evals": torch.zeros(B, dtype=torch.long)}, (shapes, None))
    expected = per_sample_vjps(f, [f.w, f.b], t, y, adj)
    assert out.shape == state.shape
    torch.testing.assert_close(out, expected, rtol=1e-12, atol=1e-14)


def test_augmented_right_hand_side_with_extra_arguments():
    A = nn.Parameter(torch.tensor(A0, dtype=torch.float64))

    class Scaled(nn.Module):
        def __init__(self):
            super().__init__()
            self.A = A

        def forward(self, t, y, scale):
            return (y @ self.A) * scale

    B = 2
    y, adj, scale = torch.tensor(Y0, dtype=torch.float64), torch.ones(B, 3, dtype=torch.float64), torch.tensor([0.5, 2.0], dtype=torch.float64)
    shapes, state = flatten_tensors(torch.zeros(B, 1, dtype=torch.float64), y, adj, torch.zeros(B, 3, 3, dtype=torch.float64))
    # per-sample argument (mapped over the batch) and shared argument (not mapped)
    mapped = AugmentedDynamicsTerm(to.ODETerm(Scaled(), with_args=True, with_stats=False), vmap_args_dims=0)
    shared = AugmentedDynamicsTerm(to.ODETerm(Scaled(), with_args=True, with_stats=False))
    with torch.no_grad():
        out = mapped.vf(torch.zeros(B, dtype=torch.float64), state, {}, (shapes, scale))
        out_shared = shared.vf(torch.zeros(B, dtype=torch.float64), state, {}, (shapes, torch.tensor(2.0, dtype=torch.float64)))
    _, dy, d_y, d_A = unflatten_tensors(shapes, out)
    torch.testing.assert_close(dy, (y @ A.detach()) * scale[:, None])
    torch.testing.assert_close(d_y, -(adj @ A.detach().T) * scale[:, None])
    torch.testing.assert_close(d_A, -torch.einsum("bi,bj->bij", y, adj) * scale[:, None, None])
    torch.testing.assert_close(unflatten_tensors(shapes, out_shared)[1][1], (y @ A.detach())[1] * 2.0)


def test_joined_batch_term_maps_time_and_scales_the_derivative():
    f = ForcedDynamics()
    inner = to.ODETerm(f)
    joined = UnwrappingODETerm(inner)
    t_start, t_end = torch.tensor([0.0, 2.0, -1.0], dtype=torch.float64), torch.tensor([3.0, 6.0, 0.5], dtype=torch.float64)
    slope = (t_end - t_start) / (t_end - t_start)[0]
    intercept = t_start - slope * t_start[0]
    y = torch.randn(3, 2, dtype=torch.float64)
    s = torch.tensor([1.2], dtype=torch.float64)  # a time on sample 0's axis, 40 % into the interval
    with torch.no_grad():
        out = joined.vf(s, y.reshape(1, -1), {"n_f_evals": torch.zeros(1, dtype=torch.long)}, (3, intercept, slope, None))
        own_t = t_start + 0.4 * (t_end - t_start)
        expected = f(own_t, y) * slope[:, None]
    assert out.shape == (1, 6)
    torch.testing.assert_close(out.reshape(3, 2), expected, rtol=1e-13, atol=1e-14)

    # and its augmented form: one reverse sweep over the joined batch
    aug = JointAugmentedDynamicsTerm(joined)
    adj = torch.randn(1, 6, dtype=torch.float64)
    shapes, state = flatten_tensors(torch.zeros(1, 1, dtype=torch.float64), y.reshape(1, -1), adj, torch.zeros(1, 2, 2, dtype=torch.float64),
                                    torch.zeros(1, 2, dtype=torch.float64))  # fmt: skip
    with torch.no_grad():
        out = aug.vf(s, state, {"n_f_evals": torch.zeros(1, dtype=torch.long)}, (shapes, (3, intercept, slope, None)))
    g = lambda tt, yy: f(torch.addcmul(intercept, slope, tt), yy[0].reshape(3, -1)).mul(slope[:, None]).reshape(1, -1)
    expected = per_sample_vjps(g, [f.w, f.b], s, y.reshape(1, -1), adj)
    torch.testing.assert_close(out, expected, rtol=1e-12, atol=1e-14)


def backsolve_with_oracle_loop(kind, t_eval):
    y0 = torch.tensor(Y0, dtype=torch.float64, requires_grad=True)
    A = nn.Parameter(torch.tensor(A0, dtype=torch.float64))
    term = to.ODETerm(LinearDynamics(A))
    ctrl = to.PIDController(1e-9, 1e-9, 0.2, 0.5, 0.0)
    if kind == "backsolve":
        adjoint = to.BacksolveAdjoint(term, to.Tsit5(), ctrl)
        adjoint.forward_adjoint = adjoint.backward_adjoint = OracleLoop()
    else:
        adjoint = to.JointBacksolveAdjoint(term, to.Tsit5(), ctrl)
        adjoint.forward_loop = adjoint.backward_loop = OracleLoop()
    if t_eval is None:
        problem = to.InitialValueProblem(y0, t_start=torch.tensor([0.0, 2.0], dtype=torch.float64), t_end=torch.tensor([3.0, 6.0], dtype=torch.float64))
    else:
        problem = to.InitialValueProblem(y0, t_eval=t_eval)
    solution = adjoint.solve(problem, term=term)
    solution.ys.mean().backward()
    return solution, y0.grad, A.grad


@pytest.mark.parametrize("kind,points", [("backsolve", T_EVAL), ("joint", T_EVAL_ALIGNED)])
def test_sweep_over_evaluation_intervals_matches_closed_form(kind, points):
    t_eval = torch.tensor(points, dtype=torch.float64)
    solution, g_y0, g_A = backsolve_with_oracle_loop(kind, t_eval)
    assert solution.ys.shape == (2, 3, 3) and len(solution.stats["backsolve"]) == 2
    want_y0, want_A = closed_form_gradients(t_eval)
    torch.testing.assert_close(g_y0, want_y0, rtol=1e-6, atol=1e-8)
    torch.testing.assert_close(g_A, want_A, rtol=1e-6, atol=1e-8)


@pytest.mark.parametrize("kind", ["backsolve", "joint"])
def test_single_backward_solve_without_evaluation_points(kind):
    solution, g_y0, g_A = backsolve_with_oracle_loop(kind, None)
    assert solution.ys.shape == (2, 1, 3) and len(solution.stats["backsolve"]) == 1
    want_y0, want_A = closed_form_gradients(torch.tensor([[0.0, 3.0], [2.0, 6.0]], dtype=torch.float64))
    # the closed form averages over both columns; column 0 is y0 itself
    y0 = torch.tensor(Y0, dtype=torch.float64)
    torch.testing.assert_close(g_y0, 2 * want_y0 - torch.full_like(y0, 1.0 / y0.numel()), rtol=1e-6, atol=1e-8)
    torch.testing.assert_close(g_A, 2 * want_A, rtol=1e-6, atol=1e-8)


def test_joint_adjoint_rejects_unaligned_evaluation_points():
    term = to.ODETerm(LinearDynamics(nn.Parameter(torch.tensor(A0))))
    adjoint = to.JointBacksolveAdjoint(term, to.Dopri5(), to.IntegralController(1e-6, 1e-6))
    problem = to.InitialValueProblem(torch.tensor(Y0), t_eval=torch.tensor(T_EVAL))
    with pytest.raises(AssertionError, match="same"):
        adjoint.solve(problem, term=term)


# ---------------------------------------------------------------------------------------------
# on the kernels (GPU)
# ---------------------------------------------------------------------------------------------


@gpu
@pytest.mark.parametrize(["dt0", "bw_dt0"], [(0.1, None), (0.2, -0.5)])
def test_backsolve_adjoint_with_fixed_step_controller(dt0, bw_dt0):
    """reference tests/adjoint_test.py:382-398"""
    y0 = torch.arange(6, dtype=torch.float, device="cuda").reshape((2, 3))
    term = to.ODETerm(LinearDynamics(nn.Parameter(torch.arange(9, device="cuda").reshape((3, 3)) / 8)))
    t_eval = torch.tensor([[0.0, 1.77, 3.0], [2.0, 3.5, 6.0]], device="cuda")
    problem = to.InitialValueProblem(y0, t_start=t_eval[:, 0], t_end=t_eval[:, -1], t_eval=t_eval)
    adjoint = to.BacksolveAdjoint(term, to.Dopri5(), to.FixedStepController())
    dt0 = torch.full((2,), dt0, device="cuda")
    bw_dt0 = torch.full((2,), bw_dt0, device="cuda") if bw_dt0 is not None else None
    solution = adjoint.solve(problem, term=term, dt0=dt0, backward_dt0=bw_dt0)
    solution.ys.mean().backward()
    grad = term.f.A.grad
    assert grad is not None and grad.shape == (3, 3) and torch.isfinite(grad).all()
    # the backward solves took the step size asked for
    width = 0.5 if bw_dt0 is not None else float(dt0[0])
    for stats, gap in zip(solution.stats["backsolve"], ([1.23, 2.5], [1.77, 1.5])):
        assert stats["n_steps"].tolist() == pytest.approx([g / width for g in gap], abs=1.01)


def make_adjoint(kind, term, atol=1e-6, rtol=0.0):
    controller = to.PIDController(atol, rtol, 0.3, 0.6, 0.0)
    cls = to.BacksolveAdjoint if kind == "backsolve" else to.JointBacksolveAdjoint
    return cls(term, to.Dopri5(), controller)


def gradcheck_inputs():
    y0 = torch.tensor(Y0, dtype=torch.double, device="cuda", requires_grad=True)
    A = nn.Parameter(torch.tensor(A0, dtype=torch.double, device="cuda", requires_grad=True))
    return y0, A


@gpu
@pytest.mark.parametrize("kind", ["backsolve", "joint-backsolve"])
def test_gradients_with_t_eval(kind):
    """reference tests/adjoint_test.py:401-442"""
    y0, A = gradcheck_inputs()
    t_eval = torch.tensor(T_EVAL_ALIGNED if kind == "joint-backsolve" else T_EVAL, dtype=torch.double, device="cuda")

    def loss(y0, params):
        term = to.ODETerm(LinearDynamics(params))
        return make_adjoint(kind, term).solve(to.InitialValueProblem(y0, t_eval=t_eval), term=term).ys.mean()

    assert torch.autograd.gradcheck(loss, (y0, A))


@gpu
@pytest.mark.parametrize("kind", ["backsolve", "joint-backsolve"])
def test_gradients_without_t_eval(kind):
    """reference tests/adjoint_test.py:445-496 (atol 1e-2 there as well: the adjoint solve does not
    see the dependence of the step sizes on the inputs)"""
    y0, A = gradcheck_inputs()
    t_start, t_end = torch.tensor([0.0, 2.0], dtype=torch.double, device="cuda"), torch.tensor([3.0, 6.0], dtype=torch.double, device="cuda")

    def loss(y0, params):
        term = to.ODETerm(LinearDynamics(params))
        problem = to.InitialValueProblem(y0, t_start=t_start, t_end=t_end, t_eval=None)
        return make_adjoint(kind, term).solve(problem, term=term).ys.mean()

    assert torch.autograd.gradcheck(loss, (y0, A), atol=1e-2)


@gpu
@pytest.mark.parametrize("kind,points", [("backsolve", T_EVAL), ("joint-backsolve", T_EVAL_ALIGNED)])
def test_gradients_match_the_closed_form(kind, points):
    y0, A = gradcheck_inputs()
    t_eval = torch.tensor(points, dtype=torch.double, device="cuda")
    term = to.ODETerm(LinearDynamics(A))
    solution = make_adjoint(kind, term, atol=1e-10, rtol=1e-10).solve(to.InitialValueProblem(y0, t_eval=t_eval), term=term)
    solution.ys.mean().backward()
    want_y0, want_A = closed_form_gradients(t_eval.cpu(), device="cuda")
    torch.testing.assert_close(y0.grad, want_y0, rtol=1e-7, atol=1e-9)
    torch.testing.assert_close(A.grad, want_A, rtol=1e-7, atol=1e-9)
    assert len(solution.stats["backsolve"]) == 2 and all(int(s["n_steps"].min()) > 3 for s in solution.stats["backsolve"])


@gpu
def test_forward_values_are_those_of_the_plain_solve_and_large_states_take_the_protocol_path():
    """A state of 40 features makes an adjoint state of 1 + 80 + 1600 columns: long rows."""
    torch.manual_seed(3)
    F, B = 40, 3
    A = nn.Parameter((torch.randn(F, F, dtype=torch.double, device="cuda") / F**0.5) - 0.5 * torch.eye(F, dtype=torch.double, device="cuda"))
    y0 = torch.randn(B, F, dtype=torch.double, device="cuda", requires_grad=True)
    t_eval = torch.tensor([[0.0, 0.5, 1.0], [0.2, 0.9, 1.3], [1.0, 1.4, 2.5]], dtype=torch.double, device="cuda")
    term = to.ODETerm(LinearDynamics(A))
    controller = to.IntegralController(1e-9, 1e-9)
    solution = to.BacksolveAdjoint(term, to.Tsit5(), controller).solve(to.InitialValueProblem(y0, t_eval=t_eval), term=term)
    with torch.no_grad():
        plain = to.AutoDiffAdjoint(to.Tsit5(), controller).solve(to.InitialValueProblem(y0.detach(), t_eval=t_eval), term=term)
    assert torch.equal(solution.ys, plain.ys) and torch.equal(solution.stats["n_steps"], plain.stats["n_steps"])
    solution.ys.square().sum().backward()

    y0_ref, A_ref = y0.detach().clone().requires_grad_(), A.detach().clone().requires_grad_()
    dts = t_eval - t_eval[:, :1]
    ys = torch.einsum("bf,befg->beg", y0_ref, torch.matrix_exp(A_ref[None, None] * dts[:, :, None, None]))
    ys.square().sum().backward()
    torch.testing.assert_close(y0.grad, y0_ref.grad, rtol=1e-6, atol=1e-7)
    torch.testing.assert_close(A.grad, A_ref.grad, rtol=1e-6, atol=1e-7)


@gpu
@pytest.mark.parametrize("name", ["mlp", "vdp"])
def test_built_in_terms_keep_parameters_as_parameters(name):
    """A built-in term built from ``nn.Parameter`` tensors holds them as parameters: optimizers find them, and the
    backsolve adjoints, which differentiate with respect to ``term.parameters()`` (reference adjoints.py:497-539), give
    about the gradient the loop's own reverse sweep gives (two discretisations of the same derivative).  (The MLP, whose
    weights the whole batch shares, through ``BacksolveAdjoint``, which calls ``f`` one sample at a time; a term with a
    parameter per sample through ``JointBacksolveAdjoint``, which calls it on the batch.)"""
    import torchode_amd.builtin_terms as bt

    torch.manual_seed(0)
    dtype, B = torch.float64, 12
    if name == "mlp":
        F, H = 6, 16
        leaves = [nn.Parameter(((torch.rand(H, F + 1, dtype=dtype) - 0.5) * 0.8).cuda()), nn.Parameter(((torch.rand(F, H, dtype=dtype) - 0.5) * 0.8).cuda())]
        f = bt.MLPField(leaves[0], torch.zeros(H, dtype=dtype, device="cuda"), leaves[1], torch.zeros(F, dtype=dtype, device="cuda"))
        y0 = (torch.rand(B, F, dtype=dtype) * 2 - 1).cuda()
    else:
        leaves = [nn.Parameter((0.5 + torch.rand(B, dtype=dtype)).cuda())]
        f = to.VanDerPol(leaves[0])
        y0 = (torch.rand(B, 2, dtype=dtype) * 2 - 1).cuda()
    assert [p is q for p, q in zip(f.parameters(), leaves)] == [True] * len(leaves)
    t_eval = torch.linspace(0, 1.0, 4, dtype=dtype, device="cuda").expand(B, 4).contiguous()
    problem = to.InitialValueProblem(y0, t_eval=t_eval)
    term = to.ODETerm(f)
    make = lambda: (to.Dopri5(), to.IntegralController(1e-9, 1e-7))
    grads = {}
    for kind in ("backsolve", "autodiff"):
        backsolve = to.BacksolveAdjoint if name == "mlp" else to.JointBacksolveAdjoint
        solver = backsolve(term, *make()) if kind == "backsolve" else to.AutoDiffAdjoint(*make())
        sol = solver.solve(problem) if kind == "backsolve" else solver.solve(problem, term)
        grads[kind] = torch.autograd.grad(sol.ys[:, -1].square().sum(), leaves)
    for a, b in zip(grads["backsolve"], grads["autodiff"]):
        assert float(b.abs().max()) > 0
        torch.testing.assert_close(a, b, rtol=1e-4, atol=1e-5 * float(b.abs().max()))

