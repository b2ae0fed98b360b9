"""Gradients through the solve loop (AutoDiffAdjoint with a y0 or parameters that require grad).

CPU: the differentiable restatement of one loop iteration (torchode_amd/autodiff.py::Replay) is
driven as a loop of its own and compared with the ATen-op oracle of the whole loop.  GPU: the
reference's gradcheck cases for this adjoint (tests/adjoint_test.py:400-496, "autodiff"), gradients
against torch autograd through the closed form y0 expm(A t), and against the backsolve adjoint.
"""
import pytest
import torch
import torch.nn as nn

import torchode_amd as to
from oracle import torch_loop
from torchode_amd import autodiff
from torchode_amd.autodiff import Replay, simulate_hits

gpu = pytest.mark.gpu
A0 = [[-1.4534, -0.3726, -0.7916], [-1.0553, 0.9511, 0.1316], [-1.8320, -0.7707, -1.0867]]
Y0 = [[0.33, 1.2, -0.4], [0.55, -0.8, 1.23]]
T_EVAL = [[0.0, 1.77, 3.0], [2.0, 3.5, 6.0]]


class LinearDynamics(nn.Module):
    def __init__(self, A):
        super().__init__()
        self.register_parameter("A", A)

    def forward(self, t, y):
        return y @ self.A


class Forced(nn.Module):
    def __init__(self):
        super().__init__()
        self.w = nn.Parameter(torch.tensor([[0.3, -1.2], [1.5, 0.1]], dtype=torch.float64))

    def forward(self, t, y):
        return torch.tanh(y @ self.w) * torch.cos(1.3 * t)[..., None] - 0.2 * y


# ---------------------------------------------------------------------------------------------
# CPU: the restated iteration against the oracle's loop
# ---------------------------------------------------------------------------------------------


def drive(replay: Replay, y0, dt0=None):
    """The loop of reference adjoints.py:50-311 around Replay.attempt / advance."""
    B = y0.shape[0]
    t_start, t_end, t_eval, direction = replay.t_start, replay.t_end, replay.t_eval, replay.direction
    f0 = replay.f(t_start, y0)
    dt = replay.first_step(y0, f0) if dt0 is None else dt0
    dt = torch.minimum(torch.maximum(dt, replay.t_lo - t_start), replay.t_hi - t_start)
    one = torch.ones(B, dtype=y0.dtype)
    state = dict(t=t_start, dt=dt, y=y0, k0=f0, prev=one, pprev=one, running=torch.ones(B, dtype=torch.bool))
    E = t_eval.shape[1]
    ys = torch.zeros(B, E, y0.shape[1], dtype=y0.dtype)
    pending = torch.ones(B, E, dtype=torch.bool)
    at_start = t_eval[:, 0] == t_start
    ys[at_start, 0] = y0[at_start]
    pending[:, 0] = ~at_start
    n_steps, n_acc = torch.zeros(B, dtype=torch.long), torch.zeros(B, dtype=torch.long)
    while True:
        attempt = replay.attempt(state)
        accept = attempt[2] < 1 if attempt[2] is not None else torch.ones(B, dtype=torch.bool)  # (no error estimate, or fixed steps)
        move = accept & state["running"]
        t_new = torch.where(move, state["t"] + state["dt"], state["t"])
        running_new = direction * t_new < direction * t_end
        hit = pending & (direction[:, None] * t_new[:, None] >= direction[:, None] * t_eval)
        idx = hit.nonzero()
        (y, k0, t, dt, prev, pprev), values = replay.advance(state, attempt, accept, running_new, (idx[:, 0], idx[:, 1]) if len(idx) else None)
        if values is not None:
            ys = ys.index_put((idx[:, 0], idx[:, 1]), values)
        pending = pending & ~hit
        n_steps += state["running"]
        n_acc += move
        state = dict(t=t, dt=dt, y=y, k0=k0, prev=prev, pprev=pprev, running=running_new)
        if not running_new.any():
            return ys, n_steps, n_acc


@pytest.mark.parametrize("method,ctrl", [
    ("dopri5", dict(kind="integral", atol=1e-6, rtol=1e-4)),
    ("tsit5", dict(kind="pid", atol=1e-7, rtol=1e-5, pcoeff=0.2, icoeff=0.5, dcoeff=0.1)),
])  # fmt: skip
def test_restated_iteration_reproduces_the_oracle_loop(method, ctrl):
    w = to.workloads.make("vdp", batch=40, dtype=torch.float64)
    w.t_eval[3, 0] = 0.25  # a first evaluation point that is not t_start
    spec = dict(ctrl)
    kind = spec.pop("kind")
    controller = to.PIDController(**spec) if kind == "pid" else to.IntegralController(**spec)
    problem = to.InitialValueProblem(w.y0, t_start=torch.zeros(40, dtype=torch.float64), t_end=w.t_eval[:, -1], t_eval=w.t_eval)
    step_method = to.Tsit5() if method == "tsit5" else to.Dopri5()
    replay = Replay(step_method, controller, to.ODETerm(w.f), None, problem, True)
    with torch.no_grad():
        ys, n_steps, n_acc = drive(replay, w.y0)
    ref = torch_loop.solve(w.f, w.y0, w.t_eval, method=method, controller=torch_loop.Controller(**ctrl), t_start=problem.t_start, t_end=problem.t_end)
    assert torch.equal(n_steps, ref["n_steps"]) and torch.equal(n_acc, ref["n_accepted"]) and (n_acc < n_steps).any()
    torch.testing.assert_close(ys, ref["ys"], rtol=1e-7, atol=1e-8)  # same operations, other association: rounding differences grow along stiff samples


@pytest.mark.parametrize("method,ctrl,first_step", [
    ("heun", dict(kind="pid", atol=1e-6, rtol=1e-4, pcoeff=0.2, icoeff=0.5, dcoeff=0.1), None),
    ("heun", dict(kind="integral", atol=1e-6, rtol=1e-4), 300.0),
    ("heun", dict(kind="fixed", atol=0.0, rtol=0.0), 400.0),
    ("euler", dict(kind="fixed", atol=0.0, rtol=0.0), 500.0),
    ("euler", dict(kind="integral", atol=1e-6, rtol=1e-4), 450.0),
])  # fmt: skip
def test_restated_iteration_reproduces_the_oracle_loop_with_heun_and_euler(method, ctrl, first_step):
    """A tableau that is neither first-same-as-last nor solution-same-as-last, the Hermite cubic and the linear
    interpolant, no error estimate (Euler) and fixed steps, against oracle/torch_loop.py::solve_low_order."""
    w = to.workloads.make("vdp", batch=40, dtype=torch.float64)
    w.t_eval[3, 0] = 0.25
    spec = dict(ctrl)
    kind = spec.pop("kind")
    controller = {"pid": to.PIDController, "integral": to.IntegralController}[kind](**spec) if kind != "fixed" else to.FixedStepController()
    t_start = torch.zeros(40, dtype=torch.float64)
    dt0 = None if first_step is None else (w.t_eval[:, -1] - t_start) / (first_step + torch.arange(40, dtype=torch.float64) % 7)
    problem = to.InitialValueProblem(w.y0, t_start=t_start, t_end=w.t_eval[:, -1], t_eval=w.t_eval)
    step_method = to.Heun() if method == "heun" else to.Euler()
    replay = Replay(step_method, controller, to.ODETerm(w.f), None, problem, True, dt0)
    with torch.no_grad():
        ys, n_steps, n_acc = drive(replay, w.y0, dt0)
    ref = torch_loop.solve_low_order(w.f, w.y0, w.t_eval, method=method, controller=torch_loop.Controller(**ctrl), t_start=t_start, t_end=problem.t_end, dt0=dt0)
    assert torch.equal(n_steps, ref["n_steps"]) and torch.equal(n_acc, ref["n_accepted"])
    assert (n_acc < n_steps).any() == (method == "heun" and kind != "fixed")
    torch.testing.assert_close(ys, ref["ys"], rtol=1e-7, atol=1e-8)


def test_recorded_times_give_back_the_evaluation_schedule():
    t_eval = torch.tensor([[0.0, 0.5, 1.0, 2.0], [1.0, 0.6, 0.2, 0.0]])
    problem = to.InitialValueProblem(torch.zeros(2, 1), t_eval=t_eval)
    replay = Replay(to.Dopri5(), to.IntegralController(1e-3, 1e-3), to.ODETerm(lambda t, y: y), None, problem, True)
    times = [[0.0, 1.0], [0.4, 0.7], [0.4, 0.1], [1.2, 0.0], [2.0, 0.0]]  # sample 0 has a rejected step, sample 1 runs backwards
    hits = simulate_hits(replay, [dict(t=torch.tensor(t)) for t in times], 4)
    got = [None if h is None else sorted(zip(h[0].tolist(), h[1].tolist())) for h in hits]
    assert got == [None, [(1, 1), (1, 2)], [(0, 1), (0, 2), (1, 3)], [(0, 3)]]
    # without evaluation points: the end point, by the last iteration, for every sample
    none = simulate_hits(replay, [dict(t=torch.tensor(t)) for t in times], 0)
    assert none[:3] == [None, None, None] and none[3][0].tolist() == [0, 1] and none[3][1] is None


# ---------------------------------------------------------------------------------------------
# GPU
# ---------------------------------------------------------------------------------------------


def closed_form(y0, A, t_eval):
    dts = t_eval - t_eval[:, :1]
    return torch.einsum("bf,befg->beg", y0, torch.matrix_exp(A[None, None] * dts[:, :, None, None]))


def inputs():
    y0 = torch.tensor(Y0, dtype=torch.double, device="cuda", requires_grad=True)
    A = nn.Parameter(torch.tensor(A0, dtype=torch.double, device="cuda"))
    return y0, A


@gpu
def test_gradients_with_t_eval():
    """reference tests/adjoint_test.py:401-442, adjoint = "autodiff" """
    y0, A = inputs()
    t_eval = torch.tensor(T_EVAL, dtype=torch.double, device="cuda")

    def loss(y0, params):
        term = to.ODETerm(LinearDynamics(params))
        adjoint = to.AutoDiffAdjoint(to.Dopri5(), to.PIDController(1e-6, 0.0, 0.3, 0.6, 0.0))
        return adjoint.solve(to.InitialValueProblem(y0, t_eval=t_eval), term=term).ys.mean()

    assert torch.autograd.gradcheck(loss, (y0, A))


@gpu
def test_gradients_without_t_eval():
    """reference tests/adjoint_test.py:445-496, adjoint = "autodiff": passes only with the gradient
    through the step sizes, there as here"""
    y0, A = inputs()
    t_start, t_end = torch.tensor([0.0, 2.0], dtype=torch.double, device="cuda"), torch.tensor([3.0, 6.0], dtype=torch.double, device="cuda")

    def loss(through):
        def fn(y0, params):
            term = to.ODETerm(LinearDynamics(params))
            adjoint = to.AutoDiffAdjoint(to.Dopri5(), to.PIDController(1e-6, 0.0, 0.3, 0.6, 0.0), backprop_through_step_size_control=through)
            return adjoint.solve(to.InitialValueProblem(y0, t_start=t_start, t_end=t_end, t_eval=None), term=term).ys.mean()

        return fn

    assert torch.autograd.gradcheck(loss(True), (y0, A), atol=1e-5)
    assert torch.autograd.gradcheck(loss(False), (y0, A), atol=1e-2)


@gpu
@pytest.mark.parametrize("method,controller", [
    (to.Dopri5, lambda: to.IntegralController(1e-10, 1e-10)),
    (to.Tsit5, lambda: to.PIDController(1e-10, 1e-10, 0.2, 0.5, 0.1)),
])  # fmt: skip
def test_gradients_match_the_closed_form(method, controller):
    y0, A = inputs()
    t_eval = torch.tensor(T_EVAL, dtype=torch.double, device="cuda")
    term = to.ODETerm(LinearDynamics(A))
    solution = to.AutoDiffAdjoint(method(), controller()).solve(to.InitialValueProblem(y0, t_eval=t_eval), term=term)
    assert solution.ys.requires_grad and (solution.stats["n_accepted"] > 10).all() and solution.stats["n_f_evals"].device.type == "cpu"
    weights = torch.linspace(0.5, 1.5, solution.ys.numel(), dtype=torch.double, device="cuda").reshape(solution.ys.shape)
    (solution.ys * weights).sum().backward()
    y0_ref, A_ref = y0.detach().clone().requires_grad_(), A.detach().clone().requires_grad_()
    (closed_form(y0_ref, A_ref, t_eval) * weights).sum().backward()
    torch.testing.assert_close(y0.grad, y0_ref.grad, rtol=1e-7, atol=1e-8)
    torch.testing.assert_close(A.grad, A_ref.grad, rtol=1e-7, atol=1e-8)
    # the values are those of the solve without grad
    with torch.no_grad():
        plain = to.AutoDiffAdjoint(method(), controller()).solve(to.InitialValueProblem(y0.detach(), t_eval=t_eval), term=term)
    assert torch.equal(plain.ys, solution.ys.detach()) and torch.equal(plain.stats["n_steps"], solution.stats["n_steps"])


@gpu
def test_parameter_gradients_agree_with_the_backsolve_adjoint_and_float32_runs():
    torch.manual_seed(1)
    f = Forced().cuda()
    y0 = torch.randn(6, 2, dtype=torch.double, device="cuda")  # does not require grad: only the parameters do
    t_eval = torch.linspace(0, 2, 5, dtype=torch.double, device="cuda").repeat(6, 1) + torch.arange(6, dtype=torch.double, device="cuda")[:, None] * 0.1
    term = to.ODETerm(f)
    ctrl = lambda: to.IntegralController(1e-9, 1e-9)
    to.AutoDiffAdjoint(to.Tsit5(), ctrl()).solve(to.InitialValueProblem(y0, t_eval=t_eval), term=term).ys.square().sum().backward()
    through_loop = f.w.grad.clone()
    f.w.grad = None
    to.BacksolveAdjoint(term, to.Tsit5(), ctrl()).solve(to.InitialValueProblem(y0, t_eval=t_eval), term=term).ys.square().sum().backward()
    torch.testing.assert_close(through_loop, f.w.grad, rtol=1e-5, atol=1e-7)
    # float32, large batch, rejected steps, both directions of time
    f32 = Forced().cuda().float()
    y0 = torch.randn(500, 2, device="cuda", requires_grad=True)
    t_eval = torch.linspace(0, 3, 7, device="cuda").repeat(500, 1)
    t_eval[::2] = t_eval[::2].flip(1)
    sol = to.AutoDiffAdjoint(to.Dopri5(), to.PIDController(1e-5, 1e-4, 0.2, 0.5, 0.0)).solve(to.InitialValueProblem(y0, t_eval=t_eval), term=to.ODETerm(f32))
    sol.ys[:, -1].sum().backward()
    assert torch.isfinite(y0.grad).all() and torch.isfinite(f32.w.grad).all() and (sol.stats["n_accepted"] < sol.stats["n_steps"]).any()


@gpu
def test_gradients_reach_tensors_inside_args():
    """The reference's loop is torch operations, so a tensor handed to `f` through `args` gets its
    gradient like any other input (adjoints.py:42-48, terms.py: `f(t, y, args)`).  Here: the system
    matrix and a scale as a dict in `args`, one of them not a leaf, no parameters on the term."""
    y0, A = inputs()
    A = A.detach().clone().requires_grad_()
    log_scale = torch.tensor(0.25, dtype=torch.double, device="cuda", requires_grad=True)
    t_eval = torch.tensor(T_EVAL, dtype=torch.double, device="cuda")
    term = to.ODETerm(lambda t, y, args: (y @ args["A"]) * args["more"][0], with_args=True)
    args = {"A": A, "more": (log_scale.exp(), "a string", 3)}
    solution = to.AutoDiffAdjoint(to.Tsit5(), to.IntegralController(1e-10, 1e-10)).solve(to.InitialValueProblem(y0, t_eval=t_eval), term=term, args=args)
    assert solution.ys.requires_grad
    weights = torch.linspace(0.5, 1.5, solution.ys.numel(), dtype=torch.double, device="cuda").reshape(solution.ys.shape)
    (solution.ys * weights).sum().backward()
    y0_ref, A_ref, ls_ref = (x.detach().clone().requires_grad_() for x in (y0, A, log_scale))
    (closed_form(y0_ref, A_ref * ls_ref.exp(), t_eval) * weights).sum().backward()
    torch.testing.assert_close(y0.grad, y0_ref.grad, rtol=1e-7, atol=1e-8)
    torch.testing.assert_close(A.grad, A_ref.grad, rtol=1e-7, atol=1e-8)
    torch.testing.assert_close(log_scale.grad, ls_ref.grad, rtol=1e-7, atol=1e-8)
    # only a tensor in args requires grad: still the differentiable path
    y0_plain = y0.detach()
    A2 = A.detach().clone().requires_grad_()
    sol = to.AutoDiffAdjoint(to.Dopri5(), to.IntegralController(1e-10, 1e-10)).solve(
        to.InitialValueProblem(y0_plain, t_eval=t_eval), term=to.ODETerm(lambda t, y, a: y @ a, with_args=True), args=A2
    )
    (sol.ys * weights).sum().backward()
    A_ref2 = A.detach().clone().requires_grad_()
    (closed_form(y0_plain, A_ref2, t_eval) * weights).sum().backward()
    torch.testing.assert_close(A2.grad, A_ref2.grad, rtol=1e-7, atol=1e-8)


def test_tensors_that_f_closes_over_are_found_from_one_evaluation():
    """CPU: captured_leaves walks the graph of f(t_start, y0) on detached inputs: a captured leaf, the leaf behind a
    captured tensor that was computed, a module's parameter and a buffer that requires grad are found; y0, the times
    and the tensors in args are not (the caller names those)."""
    from torchode_amd.autodiff import captured_leaves, wants_grad_through_term

    A = torch.tensor(A0, dtype=torch.double, requires_grad=True)
    raw = torch.tensor(0.3, dtype=torch.double, requires_grad=True)
    scale = raw.exp()  # not a leaf
    lin = nn.Linear(3, 3).double()
    lin.register_buffer("shift", torch.tensor(0.1, dtype=torch.double, requires_grad=True))
    y0 = torch.tensor(Y0, dtype=torch.double, requires_grad=True)
    problem = to.InitialValueProblem(y0, t_eval=torch.tensor(T_EVAL, dtype=torch.double))
    extra = torch.tensor(2.0, dtype=torch.double, requires_grad=True)
    term = to.ODETerm(lambda t, y, args: (y @ A) * scale + lin(y) + lin.shift + args, with_args=True)
    found = captured_leaves(term, problem, extra)
    assert {id(x) for x in found} == {id(A), id(raw), id(lin.weight), id(lin.bias), id(lin.shift)}
    assert wants_grad_through_term(term, problem, extra.detach())
    plain = to.ODETerm(lambda t, y: y @ A.detach())
    assert captured_leaves(plain, problem, None) == [] and not wants_grad_through_term(plain, problem, None)
    assert wants_grad_through_term(to.ODETerm(to.VanDerPol(torch.ones(2, requires_grad=True))), problem, None)
    assert not wants_grad_through_term(to.ODETerm(to.VanDerPol(torch.ones(2))), problem, None)


@gpu
def test_gradients_reach_tensors_that_f_closes_over_and_buffers_of_a_built_in_term():
    """The reference's loop is torch operations, so a tensor that `f` merely closes over, or a buffer behind a module,
    gets its gradient like a parameter (adjoints.py:135-260).  Here such a solve must neither take a whole-solve
    kernel (no graph) nor differentiate with respect to y0 alone."""
    y0, A = inputs()
    A = A.detach().clone().requires_grad_()
    raw = torch.tensor(0.25, dtype=torch.double, device="cuda", requires_grad=True)
    scale = raw.exp()  # captured, and not a leaf
    t_eval = torch.tensor(T_EVAL, dtype=torch.double, device="cuda")
    weights = torch.linspace(0.5, 1.5, 2 * 3 * 3, dtype=torch.double, device="cuda").reshape(2, 3, 3)
    for y_needs_grad in (True, False):
        for x in (y0, A, raw):
            x.grad = None
        y_in = y0 if y_needs_grad else y0.detach()
        term = to.ODETerm(lambda t, y: (y @ A) * scale)
        solution = to.AutoDiffAdjoint(to.Tsit5(), to.IntegralController(1e-10, 1e-10)).solve(to.InitialValueProblem(y_in, t_eval=t_eval), term=term)
        assert solution.ys.requires_grad
        (solution.ys * weights).sum().backward(retain_graph=True)
        y0_ref, A_ref, raw_ref = (x.detach().clone().requires_grad_() for x in (y0, A, raw))
        (closed_form(y0_ref, A_ref * raw_ref.exp(), t_eval) * weights).sum().backward()
        torch.testing.assert_close(A.grad, A_ref.grad, rtol=1e-7, atol=1e-8)
        torch.testing.assert_close(raw.grad, raw_ref.grad, rtol=1e-7, atol=1e-8)
        if y_needs_grad:
            torch.testing.assert_close(y0.grad, y0_ref.grad, rtol=1e-7, atol=1e-8)

    # a built-in term whose parameter requires grad: dy/dt = -k y, y(t) = y0 exp(-k t), d y / d k = -t y
    k = torch.tensor([[0.5, 1.0, 2.0], [0.3, 0.7, 1.1]], dtype=torch.double, device="cuda", requires_grad=True)
    start = y0.detach()
    sol = to.AutoDiffAdjoint(to.Dopri5(), to.IntegralController(1e-11, 1e-11)).solve(to.InitialValueProblem(start, t_eval=t_eval), term=to.ODETerm(to.LinearDecay(k)))
    assert sol.ys.requires_grad  # (without the check of the buffers this solve ran in the whole-solve kernel)
    (sol.ys * weights).sum().backward()
    elapsed = (t_eval - t_eval[:, :1])[:, :, None]
    expect = (-elapsed * start[:, None, :] * torch.exp(-k.detach()[:, None, :] * elapsed) * weights).sum(1)
    torch.testing.assert_close(k.grad, expect, rtol=1e-6, atol=1e-8)
    with torch.no_grad():  # and without grad mode the same term takes the whole-solve kernel, same values to rounding
        fused = to.AutoDiffAdjoint(to.Dopri5(), to.IntegralController(1e-11, 1e-11)).solve(to.InitialValueProblem(start, t_eval=t_eval), term=to.ODETerm(to.LinearDecay(k)))
    assert not fused.ys.requires_grad
    torch.testing.assert_close(fused.ys, sol.ys.detach(), rtol=1e-12, atol=1e-13)


@gpu
@pytest.mark.parametrize("time_dtype,data_dtype,tol", [(torch.float32, torch.float64, 2e-5), (torch.float64, torch.float32, 2e-3)], ids=["t32-y64", "t64-y32"])
def test_gradients_with_time_and_data_in_different_dtypes(time_dtype, data_dtype, tol):
    """problems.py:44-56 allows the two dtypes to differ; the forward pass keeps them apart in the
    kernels and the reverse sweep in its torch operations."""
    y0, A = inputs()
    y0 = y0.detach().to(data_dtype).requires_grad_()
    A = nn.Parameter(A.detach().to(data_dtype))
    t_eval = torch.tensor(T_EVAL, dtype=time_dtype, device="cuda")
    seen = set()

    class Watched(LinearDynamics):
        def forward(self, t, y):
            seen.add((t.dtype, y.dtype))
            return super().forward(t, y)

    solution = to.AutoDiffAdjoint(to.Tsit5(), to.IntegralController(1e-7, 1e-7)).solve(to.InitialValueProblem(y0, t_eval=t_eval), term=to.ODETerm(Watched(A)))
    assert solution.ys.dtype == data_dtype and solution.ts.dtype == time_dtype and solution.ys.requires_grad
    solution.ys.square().sum().backward()
    assert seen == {(time_dtype, data_dtype)}
    y0_ref, A_ref = y0.detach().double().requires_grad_(), A.detach().double().requires_grad_()
    closed_form(y0_ref, A_ref, t_eval.double()).square().sum().backward()
    torch.testing.assert_close(y0.grad.double(), y0_ref.grad, rtol=tol, atol=tol)
    torch.testing.assert_close(A.grad.double(), A_ref.grad, rtol=tol, atol=tol)


@gpu
@pytest.mark.parametrize("method", [to.Dopri5, to.Tsit5])
def test_gradients_with_fixed_steps(method):
    """Fixed steps (step_size_controllers.py:116-167) through the loop: the step sizes are constants, the
    gradient is that of the Runge-Kutta map itself and agrees with the closed form to the method's error."""
    y0, A = inputs()
    t_eval = torch.tensor(T_EVAL, dtype=torch.double, device="cuda")
    dt0 = torch.tensor([0.013, 0.017], dtype=torch.double, device="cuda")
    solution = to.AutoDiffAdjoint(method(), to.FixedStepController()).solve(to.InitialValueProblem(y0, t_eval=t_eval), term=to.ODETerm(LinearDynamics(A)), dt0=dt0)
    n = solution.stats["n_steps"].tolist()  # 3 / 0.013 and 4 / 0.017 steps, one more where the sums of the steps fall short of t_end
    assert solution.ys.requires_grad and n[0] in (231, 232) and n[1] in (236, 237) and (solution.status == 0).all()
    weights = torch.linspace(0.5, 1.5, solution.ys.numel(), dtype=torch.double, device="cuda").reshape(solution.ys.shape)
    (solution.ys * weights).sum().backward()
    y0_ref, A_ref = y0.detach().clone().requires_grad_(), A.detach().clone().requires_grad_()
    (closed_form(y0_ref, A_ref, t_eval) * weights).sum().backward()
    torch.testing.assert_close(y0.grad, y0_ref.grad, rtol=1e-8, atol=1e-9)
    torch.testing.assert_close(A.grad, A_ref.grad, rtol=1e-8, atol=1e-9)


@gpu
@pytest.mark.parametrize("method,controller", [
    (to.Dopri5, lambda: to.IntegralController(1e-10, 1e-10)),
    (to.Tsit5, lambda: to.PIDController(1e-10, 1e-10, 0.2, 0.5, 0.1)),
])  # fmt: skip
def test_gradients_with_respect_to_the_times_match_the_closed_form(method, controller):
    """The reference's loop is torch operations on t_start, t_end and t_eval too.  y(t_eval) = y0 expm(A (t_eval -
    t_start)): the derivative with respect to an evaluation time is f there, with respect to t_start its negative sum,
    and t_end only decides where the last step stops."""
    y0, A = inputs()
    t_start = torch.tensor([0.0, 2.0], dtype=torch.double, device="cuda", requires_grad=True)
    t_end = torch.tensor([3.0, 6.0], dtype=torch.double, device="cuda", requires_grad=True)
    t_eval = torch.tensor([[0.4, 1.77, 2.9], [2.5, 3.5, 5.2]], dtype=torch.double, device="cuda", requires_grad=True)
    solution = to.AutoDiffAdjoint(method(), controller()).solve(to.InitialValueProblem(y0, t_start, t_end, t_eval), term=to.ODETerm(LinearDynamics(A)))
    weights = torch.linspace(0.5, 1.5, solution.ys.numel(), dtype=torch.double, device="cuda").reshape(solution.ys.shape)
    (solution.ys * weights).sum().backward()
    ref = [x.detach().clone().requires_grad_() for x in (y0, A, t_start, t_eval)]
    dts = ref[3] - ref[2][:, None]
    (torch.einsum("bf,befg->beg", ref[0], torch.matrix_exp(ref[1][None, None] * dts[:, :, None, None])) * weights).sum().backward()
    for got, want in zip((y0, A, t_start, t_eval), ref):
        torch.testing.assert_close(got.grad, want.grad, rtol=1e-7, atol=1e-8)
    assert t_end.grad is not None and t_end.grad.abs().max().item() < 1e-7  # the solution at earlier times does not depend on it
    assert t_eval.grad.abs().min().item() > 1e-3


@gpu
def test_gradcheck_with_respect_to_the_times_and_the_first_step():
    """Every time input at once, the evaluation times as one tensor from which t_start and t_end are cut (the usual
    construction: the sweep must not count the shared tensor twice), and a user's first step."""
    y0, A = inputs()
    term = to.ODETerm(LinearDynamics(A))

    def through_t_eval(t_eval, dt0):
        adjoint = to.AutoDiffAdjoint(to.Dopri5(), to.PIDController(1e-6, 0.0, 0.3, 0.6, 0.0))
        return adjoint.solve(to.InitialValueProblem(y0.detach(), t_eval=t_eval), term=term, dt0=dt0).ys[:, 1:].mean()

    t_eval = torch.tensor(T_EVAL, dtype=torch.double, device="cuda", requires_grad=True)
    dt0 = torch.tensor([0.05, 0.08], dtype=torch.double, device="cuda", requires_grad=True)
    assert torch.autograd.gradcheck(through_t_eval, (t_eval, dt0), atol=1e-5)

    def without_t_eval(t_start, t_end):
        adjoint = to.AutoDiffAdjoint(to.Tsit5(), to.IntegralController(1e-7, 1e-7))
        return adjoint.solve(to.InitialValueProblem(y0.detach(), t_start, t_end), term=term).ys.mean()

    t_start = torch.tensor([0.0, 2.0], dtype=torch.double, device="cuda", requires_grad=True)
    t_end = torch.tensor([3.0, 1.0], dtype=torch.double, device="cuda", requires_grad=True)  # the second sample backwards
    assert torch.autograd.gradcheck(without_t_eval, (t_start, t_end), atol=1e-5)
    # the end state moves with t_end by f(t_end, y(t_end)), and against t_start by the transported f(t_start, y0)
    ys = to.AutoDiffAdjoint(to.Tsit5(), to.IntegralController(1e-10, 1e-10)).solve(to.InitialValueProblem(y0.detach(), t_start, t_end), term=term).ys
    (g_end,) = torch.autograd.grad(ys.sum(), t_end)
    torch.testing.assert_close(g_end, (ys[:, 0].detach() @ A.detach()).sum(dim=1), rtol=1e-6, atol=1e-8)


@gpu
@pytest.mark.parametrize("case", ["heun-pid", "heun-integral-end-only", "heun-fixed", "euler-fixed", "euler-integral"])
def test_gradcheck_through_heun_and_euler(case):
    """The loop recorded on the operator path (a tableau without first-same-as-last slope, cubic and linear dense
    output, no error estimate for Euler): y0, the term's parameters, the evaluation times and the first step."""
    y0, A = inputs()
    method, kind = case.split("-")[0], case.split("-")[1]
    t_eval = torch.tensor(T_EVAL, dtype=torch.double, device="cuda", requires_grad=True)
    dt0 = torch.tensor([0.031, 0.047], dtype=torch.double, device="cuda", requires_grad=True)

    def loss(y0, params, t_eval, dt0):
        term = to.ODETerm(LinearDynamics(params))
        controller = {"pid": lambda: to.PIDController(1e-4, 0.0, 0.3, 0.6, 0.0), "integral": lambda: to.IntegralController(1e-4, 1e-4),
                      "fixed": to.FixedStepController}[kind]()  # fmt: skip
        adjoint = to.AutoDiffAdjoint(to.Heun() if method == "heun" else to.Euler(), controller)
        if case.endswith("end-only"):
            problem = to.InitialValueProblem(y0, t_start=t_eval[:, 0], t_end=t_eval[:, -1])
        else:
            problem = to.InitialValueProblem(y0, t_eval=t_eval)
        first = dt0 if kind == "fixed" or method == "euler" else None  # (the adaptive Heun cases choose their own)
        sol = adjoint.solve(problem, term=term, dt0=first)
        assert (sol.status == 0).all() and int(sol.stats["n_steps"].max()) > 20
        return sol.ys.mean()

    assert torch.autograd.gradcheck(loss, (y0, A, t_eval, dt0), atol=1e-5, check_undefined_grad=False)


def _gradients(solver, make_inputs, weights_seed=0, **solve_kw):
    """Gradients of a weighted sum of ys with respect to everything `make_inputs` marks, through `solver`."""
    problem, term, leaves, extra = make_inputs()
    sol = solver.solve(problem, term=term, **extra, **solve_kw)
    g = torch.Generator().manual_seed(weights_seed)
    weights = torch.randn(sol.ys.shape, generator=g, dtype=torch.float64).to(sol.ys)
    (sol.ys * weights).sum().backward()
    return [None if x.grad is None else x.grad.clone() for x in leaves], sol


@gpu
@pytest.mark.parametrize("through_control", [True, False], ids=["through-control", "steps-constant"])
@pytest.mark.parametrize("case", ["tsit5-pid", "dopri5-integral", "tsit5-pid-limits", "dopri5-fixed", "tsit5-end-only", "dopri5-pid-times", "tsit5-mixed-t32", "dopri5-mixed-t64"])
def test_reverse_kernels_agree_with_the_sweep_in_torch_operations(case, through_control):
    """The reverse of an iteration in HIP kernels (tode_step_finish_backward / tode_step_stage_backward) against the
    same iteration restated as torch operations and differentiated by autograd: gradients with respect to y0, the
    parameters of f, the evaluation times, the ends of the time range and a fixed step, in both step methods, the
    three controllers, with step limits, without evaluation points, backwards in time, and with time and data in
    different dtypes."""
    from torchode_amd import autodiff

    torch.manual_seed(3)
    B = 7
    ydt = torch.float32 if case == "dopri5-mixed-t64" else torch.float64
    tdt = torch.float32 if case == "tsit5-mixed-t32" else torch.float64

    def make_inputs():
        torch.manual_seed(11)
        f = Forced().cuda().to(ydt)
        y0 = torch.randn(B, 2, dtype=torch.float64, device="cuda").to(ydt).requires_grad_()
        t_eval = (torch.linspace(0, 2.5, 6, dtype=torch.float64, device="cuda").repeat(B, 1) + torch.arange(B, dtype=torch.float64, device="cuda")[:, None] * 0.1).to(tdt)
        t_eval[::3] = t_eval[::3].flip(1)  # every third sample runs backwards
        leaves, extra = [y0, f.w], {}
        if case == "tsit5-end-only":
            t_start, t_end = t_eval[:, 0].clone().requires_grad_(), t_eval[:, -1].clone().requires_grad_()
            problem = to.InitialValueProblem(y0, t_start=t_start, t_end=t_end)
            leaves += [t_start, t_end]
        elif case == "dopri5-pid-times":
            t_eval = t_eval.clone().requires_grad_()
            problem = to.InitialValueProblem(y0, t_eval=t_eval)
            leaves += [t_eval]
        else:
            problem = to.InitialValueProblem(y0, t_eval=t_eval)
        if case == "dopri5-fixed":
            dt0 = ((t_eval[:, -1] - t_eval[:, 0]) / 17.3).detach().requires_grad_()
            extra["dt0"] = dt0
            leaves += [dt0]
        return problem, to.ODETerm(f), leaves, extra

    method = to.Tsit5 if case.startswith("tsit5") else to.Dopri5
    if "fixed" in case:
        controller = lambda: to.FixedStepController()
    elif "limits" in case:
        controller = lambda: to.PIDController(1e-5, 1e-4, 0.2, 0.5, 0.1, dt_min=1e-3, dt_max=0.2)
    elif "integral" in case:
        controller = lambda: to.IntegralController(1e-6, 1e-5)
    else:
        controller = lambda: to.PIDController(1e-6, 1e-5, 0.2, 0.5, 0.1)
    results = {}
    for kernels in (True, False):
        solver = to.AutoDiffAdjoint(method(), controller(), backprop_through_step_size_control=through_control)
        solver.backward_kernels = kernels
        results[kernels], sol = _gradients(solver, make_inputs)
        assert autodiff.LAST_SWEEP == ("kernels" if kernels else "torch")
        assert (sol.stats["n_steps"] >= 3).all()
    single = ydt == torch.float32 or tdt == torch.float32
    for a, b in zip(results[True], results[False]):
        assert (a is None) == (b is None)
        if a is not None:
            torch.testing.assert_close(a, b, rtol=5e-3 if single else 1e-9, atol=2e-3 if single else 1e-11)  # (float32: the two sweeps round differently, and the step size control amplifies it)
            assert torch.isfinite(a).all() and a.abs().max() > 0


@gpu
@pytest.mark.parametrize("features", [64, 100, 300])
@pytest.mark.parametrize("case", ["tsit5-pid", "dopri5-integral-end-only"])
def test_reverse_kernels_on_long_rows(features, case):
    """Rows of 64 features and more: the reverse kernels run one wavefront per sample; same gradients as the sweep in
    torch operations (y0, the matrix of f, the times)."""
    from torchode_amd import autodiff

    B = 9

    def make_inputs():
        g = torch.Generator().manual_seed(features)
        W = (torch.randn((features, features), generator=g, dtype=torch.float64) / features**0.5).cuda().requires_grad_()
        y0 = torch.randn((B, features), generator=g, dtype=torch.float64).cuda().requires_grad_()
        t_eval = (torch.linspace(0, 1.5, 5, dtype=torch.float64).repeat(B, 1) * (1 + 0.1 * torch.arange(B, dtype=torch.float64)[:, None])).cuda()
        t_eval[1::2] = t_eval[1::2].flip(1)
        f = lambda t, y: torch.tanh(y @ W) * torch.cos(t)[:, None] - 0.5 * y
        if case.endswith("end-only"):
            t_start, t_end = t_eval[:, 0].clone().requires_grad_(), t_eval[:, -1].clone().requires_grad_()
            return to.InitialValueProblem(y0, t_start=t_start, t_end=t_end), to.ODETerm(f), [y0, W, t_start, t_end], {}
        t_eval.requires_grad_()
        return to.InitialValueProblem(y0, t_eval=t_eval), to.ODETerm(f), [y0, W, t_eval], {}

    method = to.Tsit5 if case.startswith("tsit5") else to.Dopri5
    controller = (lambda: to.PIDController(1e-7, 1e-6, 0.2, 0.5, 0.1)) if "pid" in case else (lambda: to.IntegralController(1e-7, 1e-6))
    results = {}
    for kernels in (True, False):
        solver = to.AutoDiffAdjoint(method(), controller())
        solver.backward_kernels = kernels
        results[kernels], sol = _gradients(solver, make_inputs)
        assert autodiff.LAST_SWEEP == ("kernels" if kernels else "torch") and (sol.stats["n_steps"] >= 3).all()
    for a, b in zip(results[True], results[False]):
        torch.testing.assert_close(a, b, rtol=1e-8, atol=1e-11)
        assert torch.isfinite(a).all() and a.abs().max() > 0


@gpu
def test_a_users_subclass_is_differentiated_on_the_operator_path():
    """(more in tests/test_protocol_autograd_gpu.py)"""
    y0, A = inputs()
    term = to.ODETerm(LinearDynamics(A))
    t_eval = torch.tensor(T_EVAL, dtype=torch.double, device="cuda")

    class OwnHeun(to.Heun):  # a user's subclass: its protocol methods may do anything
        pass

    solution = to.AutoDiffAdjoint(OwnHeun(), to.IntegralController(1e-6, 1e-6)).solve(to.InitialValueProblem(y0, t_eval=t_eval), term=term)
    solution.ys.sum().backward()
    assert torch.isfinite(y0.grad).all() and torch.isfinite(A.grad).all() and A.grad.abs().max() > 0
    with torch.no_grad():  # no graph asked for: same values
        plain = to.AutoDiffAdjoint(OwnHeun(), to.IntegralController(1e-6, 1e-6)).solve(to.InitialValueProblem(y0, t_eval=t_eval), term=term)
    assert torch.equal(plain.ys, solution.ys.detach())


# ---------------------------------------------------------------------------------------------
# A differentiable solve with a built-in term: the forward pass stays in the whole-solve kernels, and the general
# kernel writes the record of the loop state that the reverse sweep starts from.  The per-step kernels' record of the
# same solve (the term behind a plain callable) is the checker: every entry, every bit.
# ---------------------------------------------------------------------------------------------


@gpu
@pytest.mark.parametrize("case", ["vdp-f32", "vdp-f64", "lorenz-f32", "linear-decay-f64", "vdp-t64-y32", "vdp-t32-y64", "max-steps", "non-monotone", "dt0",
                                  "end-only", "backwards", "limits", "non-finite"])  # fmt: skip
def test_record_of_the_whole_solve_kernel_equals_the_per_step_record(case):
    from torchode_amd.autodiff import LoopRecord

    name = "lorenz" if case.startswith("lorenz") else ("linear_decay" if case.startswith("linear") else "vdp")
    data_dtype = torch.float64 if case in ("vdp-f64", "linear-decay-f64", "vdp-t32-y64") else torch.float32
    time_dtype = {"vdp-t64-y32": torch.float64, "vdp-t32-y64": torch.float32}.get(case, data_dtype)
    w = to.workloads.make(name, batch=150, dtype=torch.float64)
    params = w.f.builtin_params().to(data_dtype)
    f = type(w.f)(params[:, 0] if params.shape[1] == 1 and name != "linear_decay" else params).cuda()
    y0, t_eval = w.y0.clone(), w.t_eval.clone()
    t_start = t_end = dt0 = None
    kw, ctrl = {}, dict(w.controller)
    if case == "max-steps":
        kw["max_steps"] = 25
    if case == "non-monotone":
        t_eval[::5, 3], t_eval[::5, 7] = t_eval[::5, 7].clone(), t_eval[::5, 3].clone()
    if case == "dt0":
        dt0 = torch.full((150,), 1e-3, dtype=time_dtype, device="cuda")
    if case == "end-only":
        t_start, t_end, t_eval = t_eval[:, 0].clone(), t_eval[:, -1].clone(), None
    if case == "backwards":
        t_eval[::2] = t_eval[::2].flip(1)
        t_eval[::2] = t_eval[::2, :1] - 0.01 * (t_eval[::2, :1] - t_eval[::2])
    if case == "limits":
        ctrl.update(dt_min=2e-2, dt_max=0.25)
    if case == "non-finite":
        y0[7] = float("inf")
    mv = lambda x, dt: None if x is None else x.to(dt).cuda()
    problem = to.InitialValueProblem(mv(y0, data_dtype), mv(t_start, time_dtype), mv(t_end, time_dtype), mv(t_eval, time_dtype))
    kind = ctrl.pop("kind")
    controller = to.PIDController(**ctrl) if kind == "pid" else to.IntegralController(**ctrl)
    solver = to.AutoDiffAdjoint({"tsit5": to.Tsit5, "dopri5": to.Dopri5}[w.method](), controller, **kw)
    whole, steps = LoopRecord(), LoopRecord()
    with torch.no_grad():
        sol_whole = solver._solve_persistent(problem, to.ODETerm(f), dt0, record=whole)
        sol_steps = solver._solve_stepwise(problem, to.ODETerm(lambda t, y: f(t, y)), dt0, None, record=steps)
    assert sol_whole is not None and whole.iterations == steps.iterations
    assert whole.iterations > 5 or case == "non-finite"  # (an infinite start value stops the whole batch after its first iteration)
    assert torch.equal(sol_whole.stats["n_steps"], sol_steps.stats["n_steps"]) and torch.equal(sol_whole.status, sol_steps.status)

    def same_record(whole):
        a, b = whole.trimmed(whole.iterations), steps.trimmed(steps.iterations)
        assert len(a) == len(b) == whole.iterations + 1
        for i, (sa, sb) in enumerate(zip(a, b)):
            for key in LoopRecord.FIELDS:
                x, y = sa[key], sb[key]
                assert x.dtype == y.dtype and x.shape == y.shape, (i, key)
                assert bool(((x == y) | ((x != x) & (y != y))).all()), (i, key, (x.double() - y.double()).abs().nan_to_num().max().item())

    same_record(whole)
    if case == "max-steps":
        assert (sol_whole.status == 3).any()
    if case == "non-finite":
        assert (sol_whole.status != 0).any()
    # The same solver again: it now knows how many entries such a record takes, and where the batch is in the
    # single-wavefront kernel's case that kernel writes the solve and the record in one launch (no flag words left
    # behind by a second pass).  Then with a record sized far too short, which sends it the long way again.
    # Both kernels that can do so are asked: the two-wavefront kernel's stepper (the choice for a batch of this size) and
    # the single-wavefront kernel.
    from torchode_amd import _lib

    in_one_kernel_case = case in ("vdp-f32", "vdp-f64", "lorenz-f32", "linear-decay-f64", "dt0", "backwards")
    # (its hand-over records of four float64 features do not fit the LDS share of a workgroup: the other kernel's case)
    two_wavefronts = in_one_kernel_case and case != "linear-decay-f64"
    known = dict(solver._record_entries)
    for variant, entries, one_kernel in ((0, None, in_one_kernel_case), (1, None, in_one_kernel_case), (2, None, two_wavefronts), (0, 3, False)):
        solver._record_entries = dict(known) if entries is None else {shape: entries for shape in known}
        again = LoopRecord()
        _lib.set_fast_kernel_variant(variant)
        try:
            with torch.no_grad():
                sol_again = solver._solve_persistent(problem, to.ODETerm(f), dt0, record=again)
        finally:
            _lib.set_fast_kernel_variant(0)
        assert (again.flags is None) == one_kernel, (variant, entries, again.flags)
        if one_kernel:
            assert _lib.last_solve_kernel_name() == ("tode::solve_pair_kernel" if variant != 1 and two_wavefronts else "tode::solve_fast_kernel"), variant
        assert again.iterations == steps.iterations
        E_ = sol_whole.ys.shape[1]
        written = (torch.arange(E_, device="cuda")[None, :] < sol_whole.stats["n_initialized"][:, None])[:, :, None] if t_eval is not None else True
        blank = lambda ys: torch.where(written, ys, torch.zeros_like(ys)) if t_eval is not None else ys
        for x, y in ((blank(sol_again.ys), blank(sol_whole.ys)), (sol_again.status, sol_whole.status)) + tuple((sol_again.stats[k], sol_whole.stats[k]) for k in sol_whole.stats):
            assert bool(((x == y) | ((x != x) & (y != y))).all())
        same_record(again)


@gpu
@pytest.mark.parametrize("through_control", [True, False], ids=["through-control", "steps-constant"])
@pytest.mark.parametrize("case", ["vdp-f64", "vdp-f32", "lorenz-f64", "linear-decay-f64", "vdp-dopri5-integral", "end-only", "times", "dt0", "dt0-constant", "max-steps", "backwards",
                                  "non-monotone", "limits"])  # fmt: skip
def test_whole_sweep_kernel_agrees_with_the_per_iteration_kernels_and_the_torch_sweep(case, through_control):
    """A differentiable solve with a built-in term three ways: the reverse sweep in one kernel (the right-hand side's
    vector-Jacobian product in closed form), the per-iteration reverse kernels with autograd through the term's torch
    forward, and the sweep in torch operations -- all from the record the whole-solve kernel wrote."""
    import torchode_amd.autodiff as autodiff

    name = "lorenz" if case.startswith("lorenz") else ("linear_decay" if case.startswith("linear") else "vdp")
    dtype = torch.float32 if case == "vdp-f32" else torch.float64
    w = to.workloads.make(name, batch=48, dtype=dtype)
    table = w.f.builtin_params().cuda()
    leaf = (table[:, 0] if name != "linear_decay" else table).clone().requires_grad_()
    y0 = w.y0.cuda().requires_grad_()
    t_eval = w.t_eval.cuda().clone()
    if case == "backwards":
        t_eval[::2] = t_eval[::2].flip(1)
        t_eval[::2] = t_eval[::2, :1] - 0.01 * (t_eval[::2, :1] - t_eval[::2])
    if case == "non-monotone":  # (every fifth row: two points swapped, written by other iterations than their neighbours)
        t_eval[::5, 3], t_eval[::5, 7] = t_eval[::5, 7].clone(), t_eval[::5, 3].clone()
    if case == "times":
        t_eval.requires_grad_()
    # (a first step large enough for its error estimate to stand above rounding: with 1e-3 even the two older sweeps
    # differ by 6e-3 in the gradient of the first step)
    # ("dt0-constant": the first step is given and no time wants a gradient, so the one-kernel sweep also reverses the
    # start of the loop, where the cotangent of the first step then ends)
    dt0 = torch.full((48,), 5e-2, dtype=dtype, device="cuda", requires_grad=case == "dt0") if case.startswith("dt0") else None
    ctrl = dict(w.controller)
    kind = ctrl.pop("kind")
    method = {"tsit5": to.Tsit5, "dopri5": to.Dopri5}[w.method]
    if case == "vdp-dopri5-integral":
        method, kind, ctrl = to.Dopri5, "integral", dict(atol=1e-6, rtol=1e-4)
    if case == "limits":
        ctrl.update(dt_min=1e-3, dt_max=0.1)
    make_controller = lambda: to.PIDController(**ctrl) if kind == "pid" else to.IntegralController(**ctrl)
    if case == "end-only":
        problem = to.InitialValueProblem(y0, t_eval[:, 0].clone(), t_eval[:, -1].clone())
    else:
        problem = to.InitialValueProblem(y0, t_eval=t_eval)
    E = problem.n_evaluation_points
    weights = torch.linspace(0.5, 1.5, max(E, 1) * y0.shape[1], dtype=dtype, device="cuda").reshape(1, max(E, 1), -1)
    wrt = [y0, leaf] + ([t_eval] if case == "times" else []) + ([dt0] if case == "dt0" else [])
    results = {}
    # ("whole-lists": the one-kernel sweep with the lists of evaluation points by iteration made by torch operations and
    # handed in, where "whole" lets the library's two kernels make them: the same bits)
    for sweep in ("whole", "whole-lists", "kernels", "torch"):
        solver = to.AutoDiffAdjoint(method(), make_controller(), max_steps=30 if case == "max-steps" else None,
                                    backprop_through_step_size_control=through_control)  # fmt: skip
        solver.backward_whole_kernel = sweep.startswith("whole")
        solver.backward_points_in_torch = sweep == "whole-lists"
        solver.backward_kernels = sweep != "torch"
        sol = solver.solve(problem, to.ODETerm(type(w.f)(leaf)), dt0=dt0)
        assert sol.ys.requires_grad
        written = (torch.arange(max(E, 1), device="cuda")[None, :] < sol.stats["n_initialized"][:, None])[:, :, None]
        if case == "non-monotone":  # (every point of every row is written here: the solves run to their ends)
            assert (sol.status == 0).all()
            written = torch.ones_like(written)
        loss = (torch.where(written, sol.ys, torch.zeros_like(sol.ys)) * weights).sum()
        results[sweep] = torch.autograd.grad(loss, wrt, allow_unused=True)
        assert autodiff.LAST_SWEEP == sweep.split("-")[0]
    if case == "max-steps":
        assert (sol.status == 3).any()
    # float64: the sweeps differ in the order of their sums only; float32: a gradient that passes through the
    # controller's powers of rounding-level error ratios is ill-conditioned, both are equally far from a float64 run
    # (through the step size rule the closed-form and autograd's products of f, equal to a few last places, are
    # amplified like any other rounding difference: measured 1e-9 of the largest gradient)
    rtol, atol = ((1e-6, 1e-6) if through_control else (1e-9, 1e-11)) if dtype == torch.float64 else (5e-3, 2e-3)
    for g, ref in zip(results["whole"], results["whole-lists"]):
        assert (g is None) == (ref is None) and (g is None or bool(((g == ref) | (g.isnan() & ref.isnan())).all()))
    for other in ("kernels", "torch"):
        for g, ref in zip(results["whole"], results[other]):
            assert (g is None) == (ref is None)
            if g is not None:
                scale = ref.abs().max().clamp_min(1.0)
                if dtype == torch.float32 and through_control:
                    # (single precision through the controller's powers of rounding-level error ratios: a few samples'
                    # gradients are noise in every sweep; the bulk agrees, and nothing is far off)
                    close = torch.isclose(g / scale, ref / scale, rtol=rtol, atol=atol)
                    assert close.float().mean().item() >= 0.9 and float(((g - ref) / scale).abs().max()) < 5e-2
                else:
                    torch.testing.assert_close(g / scale, ref / scale, rtol=rtol, atol=atol)
    assert all(g is not None and bool(g.isfinite().all()) for g in results["whole"][:2])


@pytest.mark.gpu
@pytest.mark.parametrize("features", [3, 4, 8])
@pytest.mark.parametrize("method,kind", [(to.Dopri5, "integral"), (to.Dopri5, "pid"), (to.Tsit5, "integral"), (to.Tsit5, "pid")])
def test_whole_sweep_kernel_when_every_sample_has_used_up_its_points(method, kind, features):
    """Float64 rows of 3, 4 and 8 values (the kernels under the highest register pressure), evaluation points none of
    which lies at t_start, few of them: most samples have no point left for most of the reverse sweep.  Four of these
    instantiations once lost part of the parameter gradient there (a miscompiled divergent region: see
    torchode_amd/build.py::copies_ahead_of_the_exec_restore).  Against the per-iteration reverse kernels."""
    import torchode_amd.autodiff as autodiff

    B, dtype = 70, torch.float64
    g = torch.Generator().manual_seed(5)
    k = (0.3 + 2.5 * torch.rand(B, features, generator=g, dtype=dtype)).cuda()
    y0 = (torch.rand(B, features, generator=g, dtype=dtype) * 2 - 1).cuda()
    t_start = (torch.rand(B, generator=g, dtype=dtype) - 0.5).cuda()
    t_end = t_start + (1.5 * (0.5 + 0.5 * torch.rand(B, generator=g, dtype=dtype))).cuda()
    for E in (1, 3):
        t_eval = t_start[:, None] + (t_end - t_start)[:, None] * torch.linspace(1.0 / E, 1, E, dtype=dtype, device="cuda")[None, :]
        t_eval[:, -1] = t_end
        weights = torch.linspace(0.5, 1.5, E * features, dtype=dtype, device="cuda").reshape(1, E, -1)
        results = {}
        for sweep in ("whole", "kernels"):
            leaf, y = k.clone().requires_grad_(), y0.clone().requires_grad_()
            ctrl = to.IntegralController(1e-6, 1e-4) if kind == "integral" else to.PIDController(1e-6, 1e-4, 0.2, 0.5, 0.05)
            solver = to.AutoDiffAdjoint(method(), ctrl, backprop_through_step_size_control=False)
            solver.backward_whole_kernel = sweep == "whole"
            sol = solver.solve(to.InitialValueProblem(y, t_start, t_end, t_eval), to.ODETerm(to.LinearDecay(leaf)))
            results[sweep] = torch.autograd.grad((sol.ys * weights).sum(), [y, leaf])
            assert autodiff.LAST_SWEEP == sweep
        for got, want in zip(results["whole"], results["kernels"]):
            torch.testing.assert_close(got, want, rtol=1e-9, atol=1e-9 * float(want.abs().max()))
        # (and the closed form, y0 exp(-k (t - t_start)), to the solver's own accuracy)
        span = (t_eval - t_start[:, None])[:, :, None]
        exact = (weights * -span * y0[:, None, :] * torch.exp(-k[:, None, :] * span)).sum(1)
        assert float(((results["whole"][1] - exact).abs() / exact.abs().amax(dim=1, keepdim=True)).max()) < 5e-3


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.float64], ids=["f32", "f64"])
@pytest.mark.parametrize("name", ["mlp", "reaction_diffusion"])
def test_gradients_with_the_grid_and_mlp_terms(name, dtype):
    """A differentiable solve with one of the two long-row built-in terms (weights, diffusivities or y0 require grad):
    their whole-solve kernels write no record of the loop, so the forward pass takes the per-step kernels around the
    term's torch forward (it used to ask the general kernel, which does not know these terms, for the record).  The
    reverse kernels against the sweep in torch operations, and the same term hidden behind a plain callable."""
    import torchode_amd.autodiff as autodiff
    import torchode_amd.builtin_terms as bt

    g = torch.Generator().manual_seed(3)
    r = lambda *shape: torch.rand(*shape, generator=g, dtype=torch.float64).to(dtype).cuda()
    B, E = 6, 5
    if name == "mlp":
        F, H = 8, 16
        leaves = [((r(H, F + 1) - 0.5) * 0.8).requires_grad_(), ((r(F, H) - 0.5) * 0.8).requires_grad_()]
        b1, b2 = (r(H) - 0.5) * 0.1, (r(F) - 0.5) * 0.1
        make = lambda: bt.MLPField(leaves[0], b1, leaves[1], b2)
        y0 = (r(B, F) * 2 - 1).requires_grad_()
    else:
        leaves = [(r(B) * 0.3 + 0.01).requires_grad_()]
        make = lambda: to.ReactionDiffusion(leaves[0], 16)
        y0 = r(B, 256).requires_grad_()
    t_eval = (r(B, 1) * 0.5 + 0.5) * torch.linspace(0, 1, E, dtype=dtype, device="cuda")[None, :]
    weights = torch.linspace(0.5, 1.5, E * y0.shape[1], dtype=dtype, device="cuda").reshape(1, E, -1)
    results = {}
    for sweep in ("kernels", "torch", "callable"):
        f = make()
        solver = to.AutoDiffAdjoint(to.Dopri5(), to.IntegralController(1e-6, 1e-4))
        solver.backward_kernels = sweep != "torch"
        term = to.ODETerm((lambda t, y: f(t, y)) if sweep == "callable" else f)
        sol = solver.solve(to.InitialValueProblem(y0, t_eval=t_eval), term)
        assert sol.ys.requires_grad and (sol.status == 0).all()
        results[sweep] = torch.autograd.grad((sol.ys * weights).sum(), [y0, *leaves])
        assert autodiff.LAST_SWEEP == ("torch" if sweep == "torch" else "kernels")
    rtol = 1e-9 if dtype == torch.float64 else 2e-2  # (float32 through the step size rule: the sweeps differ at the level of rounding amplified by it)
    for other in ("torch", "callable"):
        for got, want in zip(results["kernels"], results[other]):
            torch.testing.assert_close(got, want, rtol=rtol, atol=rtol * float(want.abs().max()))
    assert all(bool(x.isfinite().all()) and float(x.abs().max()) > 0 for x in results["kernels"])



# ---------------------------------------------------------------------------------------------
# Where a gradient is decided by a tie rule.  The reference keeps every step inside the time range with
# torch.clamp(dt, t_min - t, t_max - t) (adjoints.py:107, 251), whose backward pass leaves the whole cotangent with
# dt where t_min - t <= dt <= t_max - t, bounds included, and hands it to a bound only where dt lies strictly beyond
# it (minimum / maximum would halve it on a tie).  And what no operation connects to ys has no gradient at all.
# ---------------------------------------------------------------------------------------------


class OwnHeunForTies(to.Heun):  # (a subclass: the operator path, whose graph nodes run torch.clamp's own backward pass)
    pass


class OwnTsit5ForTies(to.Tsit5):
    pass


def _sweeps(method):
    """(name, step method, settings of the solver) for every backward pass that takes the method."""
    if method == "heun":
        return [("torch", to.Heun, {}), ("operator-path", OwnHeunForTies, {})]
    return [("kernels", to.Tsit5, dict(backward_kernels=True)), ("torch", to.Tsit5, dict(backward_kernels=False)), ("operator-path", OwnTsit5ForTies, {})]


@gpu
@pytest.mark.parametrize("method", ["heun", "tsit5"])
def test_a_first_step_that_equals_the_time_range_keeps_its_cotangent(method):
    """One fixed step dt0 = t_end - t_start exactly: clamp(dt0, lo, hi) meets its upper bound.  By torch.clamp's rule
    d dt / d dt0 = 1 and d dt / d t_end = 0, so with the step's result y1(dt) read at x = (t_end - t_start) / dt = 1:
    dL/d dt0 = w . (dy1/ddt - p'(1) / dt), dL/d t_end = w . p'(1) / dt (p' = dt f(t_end, y1): both interpolants take the
    last slope at their end), dL/d t_start = -dL/d t_end - [dt's part: none].  Written out below with autograd over the
    step formula and torch.clamp itself; every backward pass of the library has to return the same, element by element."""
    A = torch.tensor(A0, dtype=torch.double, device="cuda")
    # (not a linear right-hand side: Heun's dense output of y' = A y depends on dt and x only through their product)
    f = lambda t, y: torch.tanh(y @ A) * (1.0 + 0.3 * t)[:, None]
    span = torch.tensor([1.0, -0.75], dtype=torch.double, device="cuda")
    results = {}
    for name, cls, settings in _sweeps(method):
        y0 = torch.tensor(Y0, dtype=torch.double, device="cuda", requires_grad=True)
        t_start = torch.tensor([0.0, 2.0], dtype=torch.double, device="cuda", requires_grad=True)
        t_end = (t_start.detach() + span).requires_grad_()
        dt0 = span.clone().requires_grad_()
        solver = to.AutoDiffAdjoint(cls(), to.FixedStepController())
        for key, value in settings.items():
            setattr(solver, key, value)
        solution = solver.solve(to.InitialValueProblem(y0, t_start=t_start, t_end=t_end), term=to.ODETerm(f), dt0=dt0)
        assert solution.stats["n_steps"].tolist() == [1, 1]
        weights = torch.tensor([[[0.5, 1.0, 1.5]], [[-1.0, 0.25, 2.0]]], dtype=torch.double, device="cuda")
        results[name] = (solution.ys.detach(), torch.autograd.grad((solution.ys * weights).sum(), [y0, t_start, t_end, dt0]))
    # by hand: the step as a formula of (y0, t_start, t_end, dt0), the clamp as the reference writes it
    y0 = torch.tensor(Y0, dtype=torch.double, device="cuda", requires_grad=True)
    t_start = torch.tensor([0.0, 2.0], dtype=torch.double, device="cuda", requires_grad=True)
    t_end = (t_start.detach() + span).requires_grad_()
    dt0 = span.clone().requires_grad_()
    dt = torch.clamp(dt0, torch.minimum(t_start, t_end) - t_start, torch.maximum(t_end, t_start) - t_start)
    h = dt[:, None]
    if method == "heun":
        k0 = f(t_start, y0)
        k1 = f(t_start + dt, y0 + h * k0)
        y1 = y0 + h * (0.5 * k0 + 0.5 * k1)
        x = ((t_end - t_start) / ((t_start + dt) - t_start))[:, None]
        gap = y0 - y1
        value = y0 + x * (h * k0 + x * ((h * (-2 * k0 - k1) - 3 * gap) + x * (h * (k0 + k1) + 2 * gap)))
    else:
        tab = to.Tsit5.TABLEAU
        ks = [f(t_start, y0)]
        for i in range(1, 7):
            ks.append(f(t_start + float(tab.c[i]) * dt, y0 + h * sum(float(tab.a[i, j]) * ks[j] for j in range(i))))
        x = ((t_end - t_start) / ((t_start + dt) - t_start))[:, None]
        rows = tab.b_other.tolist()
        value = y0 + x * (h * ks[0] + x * sum(x**p * h * sum(rows[p][s] * ks[s] for s in range(7)) for p in range(3)))
    by_hand = torch.autograd.grad((value[:, None] * weights).sum(), [y0, t_start, t_end, dt0])
    for name, (ys, grads) in results.items():
        torch.testing.assert_close(ys[:, 0], value.detach(), rtol=1e-12, atol=1e-13, msg=name)
        for got, expected, which in zip(grads, by_hand, ("y0", "t_start", "t_end", "dt0")):
            torch.testing.assert_close(got, expected, rtol=1e-9, atol=1e-11, msg=f"{name}: {which}")
    # the rule is visible: the step's own share is not zero (small for the fifth-order pair, still 10^4 times the
    # tolerance above), and halving it would move both gradients
    assert by_hand[3].abs().min() > 1e-5


@gpu
@pytest.mark.parametrize("controller", ["integral", "pid"])
def test_separate_time_tensors_with_equal_values_get_their_own_gradients(controller):
    """t_eval[:, 0] == t_start and t_eval[:, -1] == t_end as three tensors of their own: the evaluation points get
    the interpolants' time derivatives, t_start and t_end what the start rule and the clamps hand them.  All four
    backward passes (one kernel, per-iteration kernels, torch operations, operator-path graph) agree element by element."""
    results = {}
    for sweep in ("whole", "kernels", "torch", "operator-path"):
        mu = torch.tensor([0.7, 1.9, 1.2, 2.4], dtype=torch.double, device="cuda", requires_grad=True)
        y0 = torch.tensor([[0.5, -0.2], [1.0, 0.3], [-0.8, 0.6], [0.1, 0.9]], dtype=torch.double, device="cuda", requires_grad=True)
        t_start = torch.tensor([0.0, 0.5, -0.25, 1.0], dtype=torch.double, device="cuda")
        t_end = t_start + torch.tensor([1.0, -0.8, 1.3, -1.1], dtype=torch.double, device="cuda")
        t_eval = (t_start[:, None] + (t_end - t_start)[:, None] * torch.tensor([0.0, 0.3, 0.7, 1.0], dtype=torch.double, device="cuda")).clone()
        t_eval[:, 0], t_eval[:, -1] = t_start, t_end
        leaves = [x.clone().requires_grad_() for x in (t_start, t_end, t_eval)]
        ctrl = to.IntegralController(1e-7, 1e-5) if controller == "integral" else to.PIDController(1e-7, 1e-5, 0.2, 0.5, 0.05)
        solver = to.AutoDiffAdjoint(OwnTsit5ForTies() if sweep == "operator-path" else to.Tsit5(), ctrl)
        solver.backward_kernels, solver.backward_whole_kernel = sweep in ("whole", "kernels"), sweep == "whole"
        solution = solver.solve(to.InitialValueProblem(y0, *leaves), to.ODETerm(to.VanDerPol(mu)))
        weights = torch.linspace(0.5, 1.5, solution.ys.numel(), dtype=torch.double, device="cuda").reshape(solution.ys.shape)
        results[sweep] = torch.autograd.grad((solution.ys * weights).sum(), [y0, mu, *leaves])
        if sweep != "operator-path":
            assert autodiff.LAST_SWEEP == sweep
    for sweep in ("whole", "kernels", "torch"):
        for got, expected, which in zip(results[sweep], results["operator-path"], ("y0", "mu", "t_start", "t_end", "t_eval")):
            torch.testing.assert_close(got, expected, rtol=1e-7, atol=1e-9 * float(expected.abs().max()), msg=f"{sweep}: {which}")
    assert all(float(g.abs().max()) > 0 for g in results["operator-path"])


class OwnDopri5ForTies(to.Dopri5):
    """A user's subclass: the solve takes the operator path."""


class TanhField(torch.nn.Module):
    def __init__(self, n, generator):
        super().__init__()
        self.A = torch.nn.Parameter(torch.rand(n, n, generator=generator, dtype=torch.float64) - 0.5)
        self.b = torch.nn.Parameter(torch.rand(n, generator=generator, dtype=torch.float64) - 0.5)

    def forward(self, t, y):
        return torch.tanh(y @ self.A.T + self.b) - 0.3 * y + 0.1 * torch.sin(t)[:, None]


@gpu
def test_a_last_step_of_one_unit_gives_every_pass_the_same_time_gradients():
    """In some samples of this seeded batch t + (t_end - t) rounds to one unit in the last place below t_end, so the step
    that was clamped to reach t_end is followed by a step of 2**-54, and that step writes the point at t_end: the
    derivative of the point's position multiplies whatever remainder the step's dense-output coefficients carry by
    2**54.  Dopri5's coefficients cancel to the last unit there (interpolation.py:152-166); a backward pass that does not
    form them as the forward pass does, the reference's chains of add(alpha=...), puts a rounding term of opposite signs
    on t_end and t_eval[:, -1] (two tensors here) -- 135.47 on sample 6 with the sums written out term by term."""
    g = torch.Generator().manual_seed(6188)
    u = lambda lo, hi, *shape: lo + (hi - lo) * torch.rand(*shape, generator=g, dtype=torch.float64)
    B, F = 37, 8
    f = TanhField(F, g).cuda()
    sign = torch.where(torch.rand(B, generator=g) < 0.3, -1.0, 1.0).to(torch.float64)
    t_start = u(-1, 1, B)
    t_end = t_start + sign * u(0.3, 1.5, B)
    t_eval = torch.stack((t_start, t_end), dim=1)
    dt0 = u(0.01, 0.05, B) * sign
    y_first = u(-1, 1, B, F)
    results, short = {}, None
    for sweep in ("kernels", "torch", "operator-path"):
        y0 = y_first.cuda().requires_grad_()
        leaves = [x.cuda().clone().requires_grad_() for x in (t_start, t_end, t_eval)]
        solver = to.AutoDiffAdjoint(OwnDopri5ForTies() if sweep == "operator-path" else to.Dopri5(), to.IntegralController(1e-4, 1e-3),
                                    backprop_through_step_size_control=False)  # fmt: skip
        solver.backward_kernels = sweep == "kernels"
        solution = solver.solve(to.InitialValueProblem(y0, *leaves), to.ODETerm(f), dt0=dt0.cuda())
        weights = torch.linspace(0.5, 1.5, solution.ys[0].numel(), dtype=torch.double, device="cuda").reshape(1, 2, F)
        results[sweep] = torch.autograd.grad((solution.ys * weights).sum(), [y0, f.A, f.b, *leaves])
        if sweep != "operator-path":
            assert autodiff.LAST_SWEEP == sweep
        short = solution.stats["n_steps"]
    assert short.min() >= 2 and short.max() == 4  # (the samples with a fourth step took it for one unit)
    for sweep in ("kernels", "torch"):
        for got, expected, which in zip(results[sweep], results["operator-path"], ("y0", "A", "b", "t_start", "t_end", "t_eval")):
            torch.testing.assert_close(got, expected, rtol=1e-9, atol=1e-11 * float(expected.abs().max()), msg=f"{sweep}: {which}")


@gpu
def test_a_lone_evaluation_point_at_t_start_connects_nothing_but_y0():
    """t_eval = t_start[:, None]: ys is a copy of y0 (adjoints.py:121-126) and the loop writes nothing, so in the
    reference's graph the parameters and the times are not connected to ys: autograd reports them unused (None with
    allow_unused, an error without), and y0 gets the cotangent itself.  The same from every backward pass."""
    for sweep in ("whole", "kernels", "torch", "operator-path"):
        mu = torch.tensor([0.7, 1.9], dtype=torch.double, device="cuda", requires_grad=True)
        y0 = torch.tensor([[0.5, -0.2], [1.0, 0.3]], dtype=torch.double, device="cuda", requires_grad=True)
        t_start = torch.tensor([0.0, 0.5], dtype=torch.double, device="cuda", requires_grad=True)
        t_end = torch.tensor([1.0, -0.3], dtype=torch.double, device="cuda", requires_grad=True)
        t_eval = t_start.detach()[:, None].clone().requires_grad_()
        solver = to.AutoDiffAdjoint(OwnTsit5ForTies() if sweep == "operator-path" else to.Tsit5(), to.IntegralController(1e-6, 1e-5))
        solver.backward_kernels, solver.backward_whole_kernel = sweep in ("whole", "kernels"), sweep == "whole"
        solution = solver.solve(to.InitialValueProblem(y0, t_start, t_end, t_eval), to.ODETerm(to.VanDerPol(mu)))
        assert torch.equal(solution.ys[:, 0].detach(), y0.detach()) and solution.stats["n_initialized"].tolist() == [1, 1]
        weights = torch.tensor([[[0.5, 0.7]], [[-1.5, 2.0]]], dtype=torch.double, device="cuda")
        grads = torch.autograd.grad((solution.ys * weights).sum(), [y0, mu, t_start, t_end, t_eval], allow_unused=True, retain_graph=True)
        assert torch.equal(grads[0], weights[:, 0]), sweep
        assert all(g is None for g in grads[1:]), (sweep, grads[1:])
        with pytest.raises(RuntimeError, match="not have been used"):
            torch.autograd.grad((solution.ys * weights).sum(), [mu])
