"""GPU tests of the per-step path (arbitrary Python f): fused stage / finish kernels around the
user's torch right-hand side, loop state on the device.

The right-hand sides here are the built-in terms hidden behind a plain Python callable, so the
solver cannot recognise them and must take the per-step path; their torch ops round exactly like
the scalar oracle's, which makes bit-for-bit comparison against the C oracle possible.
"""
import copy

import pytest
import torch

import torchode_amd as to
from helpers import assert_identical, c_oracle_solve, make_controller, make_method

pytestmark = pytest.mark.gpu
F32, F64 = torch.float32, torch.float64


def stepwise_solve(f, y0, t_eval, method, controller, *, t_start=None, t_end=None, dt0=None, max_steps=None, calls=None, graph=None, **extra):
    dev = "cuda"
    mv = lambda x: None if x is None else x.to(dev)
    fg = copy.deepcopy(f).to(dev)

    def opaque(t, y):  # hides the built-in module from the dispatcher
        if calls is not None:
            calls.append((t, y))
        return fg(t, y)

    solver = to.AutoDiffAdjoint(make_method(method), make_controller(controller, **extra), max_steps=max_steps, graph_iterations=graph)
    problem = to.InitialValueProblem(mv(y0), mv(t_start), mv(t_end), mv(t_eval))
    return solver.solve(problem, to.ODETerm(opaque), dt0=mv(dt0))


@pytest.mark.parametrize("dtype", [F32, F64], ids=["f32", "f64"])
@pytest.mark.parametrize("name,batch", [("linear_decay", 256), ("vdp", 512), ("lorenz", 512)])
def test_workload_matches_oracle_bit_for_bit(name, batch, dtype):
    w = to.workloads.make(name, batch=batch, dtype=dtype)
    sol = stepwise_solve(w.f, w.y0, w.t_eval, w.method, w.controller)
    assert_identical(sol, c_oracle_solve(w.f, w.y0, w.t_eval, w.method, w.controller))


@pytest.mark.parametrize("method", ["dopri5", "tsit5"])
@pytest.mark.parametrize(
    "controller",
    [dict(kind="integral", atol=1e-6, rtol=1e-4), dict(kind="pid", atol=1e-5, rtol=1e-5, pcoeff=0.3, icoeff=0.4, dcoeff=0.1)],
    ids=["I", "PID"],
)
def test_every_method_controller_pair(method, controller):
    w = to.workloads.make("vdp", batch=200, dtype=F64)
    assert_identical(stepwise_solve(w.f, w.y0, w.t_eval, method, controller), c_oracle_solve(w.f, w.y0, w.t_eval, method, controller))


def test_loop_bookkeeping_cases():
    w = to.workloads.make("vdp", batch=130, dtype=F32)
    # non-monotone evaluation times (pending mask), points outside the range, user dt0
    t_eval = w.t_eval.clone()
    t_eval[5, [3, 7]] = t_eval[5, [7, 3]]
    assert_identical(stepwise_solve(w.f, w.y0, t_eval, w.method, w.controller), c_oracle_solve(w.f, w.y0, t_eval, w.method, w.controller))
    ts, te = torch.full((130,), 0.5), (w.t_eval[:, -1] * 0.9).contiguous()
    kw = dict(t_start=ts, t_end=te, dt0=torch.full((130,), 0.02))
    sol = stepwise_solve(w.f, w.y0, w.t_eval, w.method, w.controller, **kw)
    assert_identical(sol, c_oracle_solve(w.f, w.y0, w.t_eval, w.method, w.controller, **kw))
    assert sol.stats["n_f_evals"][0].item() == 1 + 6 * sol.stats["n_steps"].max().item()
    # no evaluation points
    sol = stepwise_solve(w.f, w.y0, None, w.method, w.controller, t_start=ts, t_end=te)
    assert_identical(sol, c_oracle_solve(w.f, w.y0, None, w.method, w.controller, t_start=ts, t_end=te))
    assert sol.ys.shape == (130, 1, 2)


def test_status_handling_matches_oracle():
    w = to.workloads.make("lorenz", batch=100, dtype=F64)
    full = c_oracle_solve(w.f, w.y0, w.t_eval, w.method, w.controller)
    cap = int(full["n_steps"].median())
    sol = stepwise_solve(w.f, w.y0, w.t_eval, w.method, w.controller, max_steps=cap)
    assert_identical(sol, c_oracle_solve(w.f, w.y0, w.t_eval, w.method, w.controller, max_steps=cap))
    assert (sol.status == 3).any() and (sol.status == 0).any()
    y0 = w.y0.clone()
    y0[17, 1] = float("nan")
    sol = stepwise_solve(w.f, y0, w.t_eval, w.method, w.controller)
    assert_identical(sol, c_oracle_solve(w.f, y0, w.t_eval, w.method, w.controller))
    assert sol.status[17].item() == 4 and sol.stats["n_steps"].max().item() == 1
    t_eval = w.t_eval.clone()
    t_eval[3] = t_eval[3] * 0.05
    sol = stepwise_solve(w.f, w.y0, t_eval, w.method, w.controller, dt_min=1e-9)
    assert_identical(sol, c_oracle_solve(w.f, w.y0, t_eval, w.method, w.controller, dt_min=1e-9))
    assert sol.status[3].item() == 2


def test_agrees_with_persistent_path_and_f_sees_fresh_tensors():
    w = to.workloads.make("vdp", batch=300, dtype=F32, device="cuda")
    ctrl = to.PIDController(1e-6, 1e-4, 0.2, 0.5, 0.0)
    prob = to.InitialValueProblem(w.y0, t_eval=w.t_eval)
    a = to.AutoDiffAdjoint(to.Tsit5(), ctrl).solve(prob, to.ODETerm(w.f))
    calls = []
    b = to.AutoDiffAdjoint(to.Tsit5(), ctrl).solve(prob, to.ODETerm(lambda t, y: calls.append((t, y)) or w.f(t, y)))
    assert torch.equal(a.ys, b.ys) and torch.equal(a.stats["n_steps"], b.stats["n_steps"]) and torch.equal(a.status, b.status)
    assert torch.equal(a.stats["n_f_evals"], b.stats["n_f_evals"])
    assert len(calls) >= b.stats["n_f_evals"][0].item()  # a few speculative calls after the loop ended
    ptrs = {t.data_ptr() for t, _ in calls[:8]}
    assert len(ptrs) == 8  # every evaluation got its own time tensor
    t_min, t_max = w.t_eval.min(1).values, w.t_eval.max(1).values
    for t, _ in calls[: b.stats["n_f_evals"][0].item()]:
        assert (t >= t_min).all() and (t <= t_max).all()  # reference tests/adjoint_test.py:264-292


def test_extra_args_are_passed_by_identity():
    """reference tests/extra_args_test.py:10-22"""
    seen = []

    def f(t, y, args):
        seen.append(args)
        return torch.ones_like(y)

    token = (0, True, "hello", torch.tensor([0.0, -1.0]))
    term = to.ODETerm(f, with_args=True)
    y0 = torch.tensor([[0.0, 1.0, 2.0]], device="cuda")
    t_eval = torch.tensor([[0.0, 0.2, 0.6, 1.0]], device="cuda")
    for method in (to.Dopri5, to.Tsit5):
        sol = to.AutoDiffAdjoint(method(term), to.PIDController(1e-3, 1e-3, 0.0, 1.0, 0.0)).solve(
            to.InitialValueProblem(y0, t_eval=t_eval), term, args=token
        )
        assert seen and all(a is token for a in seen)
        assert torch.allclose(sol.ys[0, -1].cpu(), torch.tensor([1.0, 2.0, 3.0]), atol=1e-5)


@pytest.mark.parametrize("ctrl", [to.PIDController(1e-5, 1e-5, 0.0, 1.0, 0.0), to.IntegralController(1e-5, 1e-5)])
def test_constant_dynamics_in_opposite_directions(ctrl):
    """reference tests/adjoint_test.py:357-368"""
    term = to.ODETerm(lambda t, y: 2 * torch.ones_like(y))
    y0 = torch.tensor([[1.0], [9.0]], device="cuda")
    t_eval = torch.tensor([[0.0, 3.0, 5.0], [2.0, 0.5, -8.0]], device="cuda")
    sol = to.AutoDiffAdjoint(to.Dopri5(), ctrl).solve(to.InitialValueProblem(y0, t_eval=t_eval), term=term)
    assert torch.allclose(sol.ys.squeeze(-1).cpu(), torch.tensor([[1.0, 7.0, 11.0], [9.0, 6.0, -11.0]]), rtol=1e-6)
    assert (sol.status == 0).all()


def test_readme_example():
    """reference README.md:42-59: exact stats of the documented example"""
    y0 = torch.tensor([[1.2], [5.0]], device="cuda")
    t_eval = torch.stack((torch.linspace(0, 5, 10), torch.linspace(3, 4, 10))).cuda()
    term = to.ODETerm(lambda t, y: -0.5 * y)
    solver = to.AutoDiffAdjoint(to.Dopri5(term=term), to.IntegralController(atol=1e-6, rtol=1e-3, term=term))
    sol = solver.solve(to.InitialValueProblem(y0=y0, t_eval=t_eval))
    assert sol.stats["n_f_evals"].tolist() == [26, 26]
    assert sol.stats["n_steps"].tolist() == [4, 2] and sol.stats["n_accepted"].tolist() == [4, 2]
    assert sol.stats["n_initialized"].tolist() == [10, 10]
    assert torch.allclose(sol.ys[0, :, 0].cpu(), 1.2 * torch.exp(-0.5 * t_eval[0].cpu()), rtol=2e-3)


# ---------------------------------------------------------------------------------------------
# iterations replayed from a HIP graph
# ---------------------------------------------------------------------------------------------


@pytest.mark.parametrize("name,batch,dtype,n", [("vdp", 512, F32, 3), ("lorenz", 300, F32, 8), ("linear_decay", 256, F64, 1), ("vdp", 200, F64, 5)])
def test_graph_replay_equals_the_eager_loop_bit_for_bit(name, batch, dtype, n):
    w = to.workloads.make(name, batch=batch, dtype=dtype)
    ref = c_oracle_solve(w.f, w.y0, w.t_eval, w.method, w.controller)
    calls = []
    for _ in range(3):  # solves in a row, each with a graph of its own, other work in between
        with torch.no_grad():  # (under grad mode f is evaluated once more, to look for captured tensors that require grad)
            sol = stepwise_solve(w.f, w.y0, w.t_eval, w.method, w.controller, graph=n, calls=calls)
        assert_identical(sol, ref)
        torch.cuda.synchronize()
        (torch.randn(1000, device="cuda") @ torch.randn(1000, device="cuda")).item()
    # f was called for the eager iterations and once more for each recorded one, not per replay
    iterations = (int(ref["n_f_evals"][0]) - 2) // 6
    assert len(calls) // 3 == 2 + 6 * (4 + n) < 2 + 6 * iterations


def test_graph_replay_with_loop_bookkeeping_cases():
    w = to.workloads.make("vdp", batch=130, dtype=F32)
    t_eval = w.t_eval.clone()
    t_eval[5, [3, 7]] = t_eval[5, [7, 3]]  # pending mask
    assert_identical(stepwise_solve(w.f, w.y0, t_eval, w.method, w.controller, graph=2), c_oracle_solve(w.f, w.y0, t_eval, w.method, w.controller))
    # max_steps stops some samples early, in the middle of a replayed chunk
    ref = c_oracle_solve(w.f, w.y0, w.t_eval, w.method, w.controller, max_steps=23)
    assert (ref["status"] == 3).any()
    assert_identical(stepwise_solve(w.f, w.y0, w.t_eval, w.method, w.controller, max_steps=23, graph=7), ref)
    # a solve that ends within the eager iterations never records a graph
    short = w.t_eval[:, :2] * 1e-3
    assert_identical(stepwise_solve(w.f, w.y0, short, w.method, w.controller, graph=4), c_oracle_solve(w.f, w.y0, short, w.method, w.controller))
    # without evaluation points
    ts, te = w.t_eval[:, 0].contiguous(), w.t_eval[:, -1].contiguous()
    ref = c_oracle_solve(w.f, w.y0, None, w.method, w.controller, t_start=ts, t_end=te)
    assert_identical(stepwise_solve(w.f, w.y0, None, w.method, w.controller, t_start=ts, t_end=te, graph=4), ref)


# ---------------------------------------------------------------------------------------------
# time and data in different dtypes (reference problems.py:44-56, tests/dtype_stability_test.py):
# the per-step kernels against the protocol path (per-call operators), which states the same
# arithmetic operator by operator -- same bits
# ---------------------------------------------------------------------------------------------


class OperatorTsit5(to.Tsit5):
    """Not recognised by the fused paths: every protocol call goes through its own kernel."""


class OperatorDopri5(to.Dopri5):
    pass


def mixed_case(case, time_dtype, data_dtype):
    """(f, y0, t_start, t_end, t_eval, dt0, method, controller keywords, max_steps) on the GPU"""
    dev = "cuda"
    g = torch.Generator().manual_seed(17)
    if case in ("wide", "rows"):  # rows of 100 values: one wavefront per sample; of 1300: one workgroup per sample in the finish kernel
        B, F = (37, 100) if case == "wide" else (11, 1300)
        rate = (0.5 + torch.rand(B, F, generator=g, dtype=torch.float64)).to(data_dtype).to(dev)
        f = lambda t, y: torch.sin(t).to(y.dtype)[:, None] - rate * y
        y0 = torch.randn(B, F, generator=g, dtype=torch.float64)
        t_eval = torch.linspace(0.0, 2.0, 9, dtype=torch.float64).repeat(B, 1) * (0.5 + torch.rand(B, 1, generator=g, dtype=torch.float64))
        name = "tsit5"
        ctrl = dict(kind="pid", atol=1e-6, rtol=1e-5, pcoeff=0.2, icoeff=0.5, dcoeff=0.1)
    else:
        w = to.workloads.make("lorenz" if case == "lorenz" else "vdp", batch=200, dtype=torch.float64)
        fd = copy.deepcopy(w.f).to(data_dtype).to(dev)
        f = lambda t, y: fd(t, y) + 1e-3 * torch.cos(t).to(y.dtype)[:, None]  # (t matters, in its own dtype)
        y0, t_eval, name, ctrl = w.y0, w.t_eval.clone(), w.method, dict(w.controller)
    t_start, t_end, dt0, max_steps = t_eval[:, 0].clone(), t_eval[:, -1].clone(), None, None
    if case == "backwards":
        t_eval[::2] = t_eval[::2].flip(1)
        t_eval[::2] = t_eval[::2, :1] - 0.01 * (t_eval[::2, :1] - t_eval[::2])  # (a short way back: no blow-up)
        t_start, t_end = t_eval[:, 0].clone(), t_eval[:, -1].clone()
    if case == "outside":  # first point after t_start, last point beyond t_end, rows not monotone
        t_start, t_end = t_eval[:, 0] - 0.25, t_eval[:, -2].clone()
        t_eval[::5, 3], t_eval[::5, 7] = t_eval[::5, 7].clone(), t_eval[::5, 3].clone()
    if case == "no-t_eval":
        t_eval = None
    if case == "dt0":
        dt0 = torch.full((y0.shape[0],), 1e-3, dtype=torch.float64)
    if case == "limits":
        ctrl.update(dt_min=2e-2, dt_max=0.25)
        max_steps = 60
    mv = lambda x, dt: None if x is None else x.to(dt).to(dev)
    return f, mv(y0, data_dtype), mv(t_start, time_dtype), mv(t_end, time_dtype), mv(t_eval, time_dtype), mv(dt0, time_dtype), name, ctrl, max_steps


@pytest.mark.parametrize("time_dtype,data_dtype", [(F64, F32), (F32, F64)], ids=["t64-y32", "t32-y64"])
@pytest.mark.parametrize("case", ["vdp", "lorenz", "wide", "rows", "backwards", "outside", "no-t_eval", "dt0", "limits"])
def test_mixed_dtypes_per_step_kernels_equal_the_operator_path(case, time_dtype, data_dtype):
    f, y0, t_start, t_end, t_eval, dt0, name, ctrl, max_steps = mixed_case(case, time_dtype, data_dtype)
    seen = []

    def rhs(t, y):
        seen.append((t.dtype, y.dtype))
        return f(t, y)

    problem = to.InitialValueProblem(y0, t_start, t_end, t_eval)
    fused_method, operator_method = {"tsit5": (to.Tsit5, OperatorTsit5), "dopri5": (to.Dopri5, OperatorDopri5)}[name]
    fused = to.AutoDiffAdjoint(fused_method(), make_controller(ctrl), max_steps=max_steps).solve(problem, to.ODETerm(rhs), dt0=dt0)
    assert set(seen) == {(time_dtype, data_dtype)}
    ops = to.AutoDiffAdjoint(operator_method(), make_controller(ctrl), max_steps=max_steps).solve(problem, to.ODETerm(rhs), dt0=dt0)
    assert fused.ys.dtype == data_dtype and fused.ts.dtype == time_dtype and fused.ys.shape == ops.ys.shape
    for key in ("n_steps", "n_accepted", "n_initialized"):
        assert torch.equal(fused.stats[key], ops.stats[key]), key
    assert torch.equal(fused.status, ops.status) and torch.equal(fused.stats["n_f_evals"], ops.stats["n_f_evals"])
    E = fused.ys.shape[1]
    written = torch.arange(E, device="cuda")[None, :] < ops.stats["n_initialized"][:, None]
    if case == "outside":  # rows that are not monotone: compare what both wrote (the reference leaves the rest unset)
        written = written & fused.ys.isfinite().all(dim=2) & ops.ys.isfinite().all(dim=2)
    a, b = fused.ys[written], ops.ys[written]
    assert bool(((a == b) | (a.isnan() & b.isnan())).all()), (a - b).abs().nan_to_num().max().item()
    assert int(fused.stats["n_steps"].max()) >= 3
    if case == "limits":
        assert (fused.status != 0).any()  # dt_min reached somewhere (status 2), or max_steps (3)
    elif case != "outside":
        assert (fused.status == 0).all()


# ---------------------------------------------------------------------------------------------
# fixed steps (reference step_size_controllers.py:116-167, tests/fixed_step_controller_test.py):
# Dopri5 / Tsit5 with the library's FixedStepController run in the per-step kernels; a subclass of
# the method sends the same solve through the operator path
# ---------------------------------------------------------------------------------------------


@pytest.mark.parametrize("time_dtype,data_dtype", [(F32, F32), (F64, F64), (F64, F32)], ids=["f32", "f64", "t64-y32"])
@pytest.mark.parametrize("case", ["vdp", "wide", "rows", "backwards", "no-t_eval", "outside"])
def test_fixed_steps_in_the_per_step_kernels_equal_the_operator_path(case, time_dtype, data_dtype):
    f, y0, t_start, t_end, t_eval, _, name, _, _ = mixed_case(case, time_dtype, data_dtype)
    B = y0.shape[0]
    span = (t_end - t_start).double()
    dt0 = (span / (40.0 + torch.arange(B, device="cuda", dtype=torch.float64) % 7 + 0.37)).to(time_dtype)  # 41 to 47 steps, the last one cut
    problem = to.InitialValueProblem(y0, t_start, t_end, t_eval)
    fused_method, operator_method = {"tsit5": (to.Tsit5, OperatorTsit5), "dopri5": (to.Dopri5, OperatorDopri5)}[name]
    fused = to.AutoDiffAdjoint(fused_method(), to.FixedStepController(), max_steps=44 if case == "outside" else None).solve(problem, to.ODETerm(f), dt0=dt0)
    ops = to.AutoDiffAdjoint(operator_method(), to.FixedStepController(), max_steps=44 if case == "outside" else None).solve(problem, to.ODETerm(f), dt0=dt0)
    for key in ("n_steps", "n_accepted", "n_initialized"):
        assert torch.equal(fused.stats[key], ops.stats[key]), key
    assert torch.equal(fused.status, ops.status) and torch.equal(fused.stats["n_f_evals"], ops.stats["n_f_evals"])
    assert torch.equal(fused.stats["n_steps"], fused.stats["n_accepted"]) and 38 <= int(fused.stats["n_steps"].min()) <= int(fused.stats["n_steps"].max()) <= 48
    E = fused.ys.shape[1]
    written = torch.arange(E, device="cuda")[None, :] < ops.stats["n_initialized"][:, None]
    if case == "outside":
        written = written & fused.ys.isfinite().all(dim=2) & ops.ys.isfinite().all(dim=2)
        assert (fused.status == 3).any()  # max_steps cuts the slower samples short
    else:
        assert (fused.status == 0).all()
    a, b = fused.ys[written], ops.ys[written]
    assert bool(((a == b) | (a.isnan() & b.isnan())).all()), (a - b).abs().nan_to_num().max().item()
    assert a.isfinite().float().mean().item() > 0.5  # (some of the stiffer samples blow up at these step sizes, in both paths alike)
    with pytest.raises(AssertionError, match="dt0"):
        to.AutoDiffAdjoint(fused_method(), to.FixedStepController()).solve(problem, to.ODETerm(f))


# ---------------------------------------------------------------------------------------------
# Heun and Euler (reference single_step_methods/heun.py, euler.py) in the per-step kernels: no
# derivative carried between steps, the step's result formed in the finish kernel, cubic / linear
# dense output, controller exponents of order 2 / 1, no error estimate for Euler.  A subclass of
# the method sends the same solve through the operator path.
# ---------------------------------------------------------------------------------------------


class OperatorHeun(to.Heun):
    pass


class OperatorEuler(to.Euler):
    pass


@pytest.mark.parametrize("time_dtype,data_dtype", [(F32, F32), (F64, F64), (F64, F32), (F32, F64)], ids=["f32", "f64", "t64-y32", "t32-y64"])
@pytest.mark.parametrize("controller", ["integral", "pid", "fixed"])
@pytest.mark.parametrize("method", ["heun", "euler"])
@pytest.mark.parametrize("case", ["vdp", "lorenz", "backwards", "outside", "no-t_eval", "dt0", "limits"])
def test_heun_and_euler_in_the_per_step_kernels_equal_the_operator_path(case, method, controller, time_dtype, data_dtype):
    f, y0, t_start, t_end, t_eval, dt0, _, ctrl, max_steps = mixed_case(case, time_dtype, data_dtype)
    B = y0.shape[0]
    if controller == "fixed" or (method == "euler" and dt0 is None and case != "vdp"):
        # (Euler under an adaptive controller keeps whatever step it starts with: one case leaves that to the start rule)
        span = (t_end - t_start).double()
        dt0 = (span / (40.0 + torch.arange(B, device="cuda", dtype=torch.float64) % 7 + 0.37)).to(time_dtype)
    if controller == "fixed":
        make = to.FixedStepController
    else:
        spec = dict(kind=controller, atol=1e-3, rtol=1e-2, **{k: ctrl[k] for k in ("dt_min", "dt_max") if k in ctrl})
        if controller == "pid":
            spec.update(pcoeff=0.2, icoeff=0.5, dcoeff=0.1)
        make = lambda: make_controller(spec)
    max_steps = 44 if case in ("outside", "limits") else 400
    calls = {"kernels": [], "operators": []}

    def rhs(which):
        def g(t, y):
            calls[which].append((t, y))
            return f(t, y)

        return g

    problem = to.InitialValueProblem(y0, t_start, t_end, t_eval)
    fused_method, operator_method = {"heun": (to.Heun, OperatorHeun), "euler": (to.Euler, OperatorEuler)}[method]
    with torch.no_grad():
        fused_solver = to.AutoDiffAdjoint(fused_method(), make(), max_steps=max_steps)
        assert fused_solver._stepwise_ok(problem, to.ODETerm(f))
        fused = fused_solver.solve(problem, to.ODETerm(rhs("kernels")), dt0=dt0)
        ops_solver = to.AutoDiffAdjoint(operator_method(), make(), max_steps=max_steps)
        assert not ops_solver._stepwise_ok(problem, to.ODETerm(f))
        ops = ops_solver.solve(problem, to.ODETerm(rhs("operators")), dt0=dt0)
    assert fused.ys.dtype == data_dtype and fused.ts.dtype == time_dtype and fused.ys.shape == ops.ys.shape
    for key in ("n_steps", "n_accepted", "n_initialized", "n_f_evals"):
        assert torch.equal(fused.stats[key], ops.stats[key]), key
    assert torch.equal(fused.status, ops.status)
    # f is called as often as the counter says (the kernels' loop runs ahead of the device by a few iterations whose
    # kernels do nothing), with tensors of its own that hold what the operator path's calls held
    n = int(ops.stats["n_f_evals"][0])
    assert len(calls["operators"]) == n and len(calls["kernels"]) >= n
    stages = 2 if method == "heun" else 1
    for i in sorted({0, 1, 2, stages * 3, n - stages - 1, n - 1} & set(range(n))):
        (ta, ya), (tb, yb) = calls["kernels"][i], calls["operators"][i]
        assert ta.dtype == time_dtype and ya.dtype == data_dtype
        running_rows = torch.isfinite(yb).all(dim=1)
        if i < n - stages:  # (in the last iteration the finished samples differ: stale in one path, frozen in the other)
            assert torch.equal(ta, tb) and torch.equal(ya[running_rows], yb[running_rows]), i
    assert len({x.data_ptr() for pair in calls["kernels"] for x in pair}) == 2 * len(calls["kernels"])
    E = fused.ys.shape[1]
    written = torch.arange(E, device="cuda")[None, :] < ops.stats["n_initialized"][:, None]
    if case == "outside":  # every fifth row is not monotone: what is written there is no prefix of the row (the counts are compared above)
        written = written & (torch.arange(B, device="cuda") % 5 != 0)[:, None]
    a, b = fused.ys[written], ops.ys[written]
    assert bool(((a == b) | (a.isnan() & b.isnan())).all()), (a - b).abs().nan_to_num().max().item()
    if case == "limits" and method == "heun" and controller != "fixed":
        assert (fused.status == 2).any()  # the smallest step allowed is too long for these tolerances
    else:
        assert int(fused.stats["n_steps"].max()) >= 3
    if method == "euler" or controller == "fixed":
        assert torch.equal(fused.stats["n_steps"], fused.stats["n_accepted"])
    elif case in ("vdp", "lorenz"):
        assert (fused.stats["n_steps"] > fused.stats["n_accepted"]).any()  # rejected steps are part of the case


@pytest.mark.parametrize("time_dtype,data_dtype", [(F32, F32), (F64, F64), (F64, F32)], ids=["f32", "f64", "t64-y32"])
@pytest.mark.parametrize("controller", ["integral", "pid", "fixed"])
@pytest.mark.parametrize("method", ["heun", "euler"])
@pytest.mark.parametrize("with_points", [True, False], ids=["t_eval", "end-only"])
@pytest.mark.parametrize("rows", ["wide", "rows"])
def test_long_rows_with_heun_and_euler_in_the_wavefront_kernels_equal_the_operator_path(rows, with_points, method, controller, time_dtype, data_dtype):
    """Rows of 100 values: one wavefront per sample in the finish kernel, which for these two methods also forms the
    step's result (each lane for the features it needs, never through memory another lane has just written); rows of
    1300: one workgroup per sample."""
    f, y0, t_start, t_end, t_eval, _, _, _, _ = mixed_case(rows, time_dtype, data_dtype)
    B = y0.shape[0]
    dt0 = None
    if controller == "fixed" or method == "euler":
        dt0 = ((t_end - t_start).double() / (40.0 + torch.arange(B, device="cuda", dtype=torch.float64) % 7 + 0.37)).to(time_dtype)
    if controller == "fixed":
        make = to.FixedStepController
    else:
        spec = dict(kind=controller, atol=1e-3, rtol=1e-2)
        if controller == "pid":
            spec.update(pcoeff=0.2, icoeff=0.5, dcoeff=0.1)
        make = lambda: make_controller(spec)
    problem = to.InitialValueProblem(y0, t_start, t_end, t_eval if with_points else None)
    fused_method, operator_method = {"heun": (to.Heun, OperatorHeun), "euler": (to.Euler, OperatorEuler)}[method]
    with torch.no_grad():
        fused_solver = to.AutoDiffAdjoint(fused_method(), make(), max_steps=300)
        assert fused_solver._stepwise_ok(problem, to.ODETerm(f))
        fused = fused_solver.solve(problem, to.ODETerm(f), dt0=dt0)
        ops_solver = to.AutoDiffAdjoint(operator_method(), make(), max_steps=300)
        assert not ops_solver._stepwise_ok(problem, to.ODETerm(f))
        ops = ops_solver.solve(problem, to.ODETerm(f), dt0=dt0)
    for key in ("n_steps", "n_accepted", "n_initialized", "n_f_evals"):
        assert torch.equal(fused.stats[key], ops.stats[key]), key
    assert torch.equal(fused.status, ops.status) and (fused.status == 0).all()
    assert fused.ys.shape == ops.ys.shape and bool((fused.ys == ops.ys).all()), (fused.ys - ops.ys).abs().max().item()
    assert int(fused.stats["n_steps"].max()) >= 10
    if method == "heun" and controller == "integral" and rows == "wide":
        assert (fused.stats["n_steps"] > fused.stats["n_accepted"]).any()  # rejected steps are part of the case


@pytest.mark.parametrize("method", ["heun", "euler"])
def test_graph_replay_with_heun_and_euler(method):
    w = to.workloads.make("vdp", batch=300, dtype=F32)
    f = copy.deepcopy(w.f).to("cuda")
    problem = to.InitialValueProblem(w.y0.to("cuda"), t_eval=w.t_eval.to("cuda"))
    dt0 = torch.full((300,), 5e-3, device="cuda")
    m = {"heun": to.Heun, "euler": to.Euler}[method]
    with torch.no_grad():
        eager = to.AutoDiffAdjoint(m(), to.IntegralController(1e-3, 1e-2)).solve(problem, to.ODETerm(f), dt0=dt0)
        replayed = to.AutoDiffAdjoint(m(), to.IntegralController(1e-3, 1e-2), graph_iterations=5).solve(problem, to.ODETerm(f), dt0=dt0)
    for key in ("n_steps", "n_accepted", "n_initialized"):
        assert torch.equal(eager.stats[key], replayed.stats[key]), key
    assert torch.equal(eager.ys, replayed.ys) and torch.equal(eager.status, replayed.status)
    assert int(eager.stats["n_steps"].max()) > 40


@pytest.mark.parametrize("seed", range(10))
def test_random_configurations_match_oracle_bit_for_bit(seed):
    """The seeded random configurations of the whole-solve suite (term, shapes, time spans, evaluation points,
    tolerances, controller coefficients) through the per-step kernels."""
    from test_persistent_gpu import _random_case

    f, y0, t_eval, t_start, t_end, method, controller = _random_case(2000 + seed)
    ref = c_oracle_solve(f, y0, t_eval, method, controller, t_start=t_start, t_end=t_end, max_steps=4000)
    assert (ref["status"] == 0).all() and 2 <= int(ref["n_steps"].max()) < 4000
    sol = stepwise_solve(f, y0, t_eval, method, controller, t_start=t_start, t_end=t_end, max_steps=4000)
    assert_identical(sol, ref)


@pytest.mark.parametrize("seed", range(200, 216))
def test_wild_configurations_match_oracle_bit_for_bit(seed):
    """tests/helpers.py::wild_case through the per-step kernels."""
    from helpers import wild_case

    f, y0, t_eval, t_start, t_end, method, ctrl, max_steps, dt0 = wild_case(seed)
    kw = dict(t_start=t_start, t_end=t_end, dt0=dt0, max_steps=max_steps)
    assert_identical(stepwise_solve(f, y0, t_eval, method, ctrl, **kw), c_oracle_solve(f, y0, t_eval, method, ctrl, **kw))


@pytest.mark.parametrize("seed", range(720, 728))
def test_controller_powers_that_are_shortcuts_match_oracle_bit_for_bit(seed):
    """tests/helpers.py::shortcut_case (controller exponents -1, 2, 3, -2, -0.5) through the per-step kernels."""
    from helpers import shortcut_case

    f, y0, t_eval, t_start, t_end, method, ctrl, max_steps, dt0 = shortcut_case(seed)
    kw = dict(t_start=t_start, t_end=t_end, dt0=dt0, max_steps=max_steps)
    assert_identical(stepwise_solve(f, y0, t_eval, method, ctrl, **kw), c_oracle_solve(f, y0, t_eval, method, ctrl, **kw))


@pytest.mark.parametrize("seed", range(500, 508))
def test_wild_configurations_with_non_finite_samples(seed):
    """wild_case with three samples NaN, infinite, huge or blowing up later (tests/helpers.py::poisoned): status 4, 2
    and 3 in every mixture and the batch-wide stop, through the per-step kernels."""
    from helpers import poisoned, wild_case

    f, y0, t_eval, t_start, t_end, method, ctrl, max_steps, dt0 = wild_case(seed)
    y0 = poisoned(y0, seed)
    kw = dict(t_start=t_start, t_end=t_end, dt0=dt0, max_steps=min(max_steps, 400))
    assert_identical(stepwise_solve(f, y0, t_eval, method, ctrl, **kw), c_oracle_solve(f, y0, t_eval, method, ctrl, **kw))


def _mixed_fixtures():
    import glob
    import os

    return sorted(glob.glob(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "*_mixed.json")))


@pytest.mark.parametrize("path", _mixed_fixtures(), ids=lambda p: p.split("/")[-1])
def test_mixed_dtypes_match_the_aten_op_oracle_fixture(path):
    """tests/golden/*_mixed.json: the reference's loop as ATen CPU operations with time and data in different dtypes,
    written in the authoring container.  The per-step kernels and the operator path reproduce every bit of them."""
    import hashlib
    import json

    g = json.load(open(path))
    time_dtype, data_dtype = getattr(torch, g["time_dtype"]), getattr(torch, g["data_dtype"])
    w = to.workloads.make(g["workload"], batch=g["batch"], dtype=torch.float64)
    params = w.f.builtin_params().to(data_dtype)
    f = type(w.f)(params[:, 0] if params.shape[1] == 1 else params).cuda()
    problem = to.InitialValueProblem(w.y0.to(data_dtype).cuda(), t_eval=w.t_eval.to(time_dtype).cuda())
    fused_method, operator_method = {"tsit5": (to.Tsit5, OperatorTsit5), "dopri5": (to.Dopri5, OperatorDopri5)}[g["method"]]
    # the per-step kernels, the operator path, and (the term handed over as it is, not behind a plain callable) the
    # general whole-solve kernel, which is built for the four (time, data) pairs
    for method, term in ((fused_method, to.ODETerm(lambda t, y: f(t, y))), (operator_method, to.ODETerm(lambda t, y: f(t, y))), (fused_method, to.ODETerm(f))):
        solver = to.AutoDiffAdjoint(method(), make_controller(g["controller"]))
        assert solver._persistent_ok(problem, term) == (term.f is f)
        with torch.no_grad():
            sol = solver.solve(problem, term)
        for key in ("n_steps", "n_accepted", "n_initialized"):
            assert sol.stats[key].tolist() == g[key], (method.__name__, key)
        assert sol.status.tolist() == g["status"] and int(sol.stats["n_f_evals"][0]) == g["n_f_evals"]
        ys = sol.ys.cpu()
        assert ys.dtype == data_dtype and sol.ts.dtype == time_dtype
        assert [float(v).hex() for v in ys[g["subset"]].flatten().tolist()] == g["ys_subset"], method.__name__
        assert hashlib.sha256(ys.contiguous().numpy().tobytes()).hexdigest() == g["ys_sha256"], method.__name__


def _fixed_fixtures():
    import glob
    import os

    return sorted(glob.glob(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "*_fixed.json")))


@pytest.mark.parametrize("path", _fixed_fixtures(), ids=lambda p: p.split("/")[-1])
def test_fixed_steps_match_the_aten_op_oracle_fixture(path):
    """tests/golden/*_fixed.json: the reference's loop with its FixedStepController as ATen CPU operations, written in
    the authoring container.  The per-step kernels and the operator path reproduce every bit of them."""
    import hashlib
    import json

    g = json.load(open(path))
    dtype = getattr(torch, g["dtype"])
    w = to.workloads.make(g["workload"], batch=g["batch"], dtype=dtype)
    span = (w.t_eval[:, -1] - w.t_eval[:, 0]).double()
    dt0 = (span / (60.37 + torch.arange(g["batch"], dtype=torch.float64) % 7)).to(dtype).cuda()
    f = copy.deepcopy(w.f).cuda()
    problem = to.InitialValueProblem(w.y0.cuda(), t_eval=w.t_eval.cuda())
    fused_method, operator_method = {"tsit5": (to.Tsit5, OperatorTsit5), "dopri5": (to.Dopri5, OperatorDopri5)}[g["method"]]
    for method in (fused_method, operator_method):
        sol = to.AutoDiffAdjoint(method(), to.FixedStepController()).solve(problem, to.ODETerm(lambda t, y: f(t, y)), dt0=dt0)
        for key in ("n_steps", "n_accepted", "n_initialized"):
            assert sol.stats[key].tolist() == g[key], (method.__name__, key)
        assert sol.status.tolist() == g["status"] and int(sol.stats["n_f_evals"][0]) == g["n_f_evals"]
        ys = sol.ys.cpu()
        assert [float(v).hex() for v in ys[g["subset"]].flatten().tolist()] == g["ys_subset"], method.__name__
        clean = ys.nan_to_num(nan=0.0, posinf=float("inf"), neginf=float("-inf"))
        assert hashlib.sha256(clean.contiguous().numpy().tobytes()).hexdigest() == g["ys_sha256_nan_as_zero"], method.__name__
