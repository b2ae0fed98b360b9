"""Seeded comparisons over configurations drawn at random, each kernel path against the path or oracle that pins it:

* time spans whose ends differ in sign and scale (samples that land one unit in the last place short of or past t_end,
  final states near the top of the dtype's range) through every whole-solve dispatch, against the C oracle: same bits;
* the reaction-diffusion and MLP kernels (grids of 16 to 128 cells a side, 3 to 64 state values, with and without
  evaluation points) against the protocol path (grid: same bits; MLP: the tolerance of its tests);
* time and data in different dtypes, general kernel against per-step kernels: same bits;
* Heun and Euler, per-step kernels against the operator path: same bits;
* the one-kernel reverse sweep (its record from the recording whole-solve kernel) against the sweep in torch operations.

The same generators were run once over several thousand seeds each; what they found is in the tests their findings
left behind (test_persistent_gpu.py, test_autodiff.py).  Here a few dozen seeds of each run with the suite."""
import pytest
import torch

import torchode_amd as to
from helpers import assert_identical, c_oracle_solve, gpu_solve, make_controller, poisoned, wild_case

pytestmark = pytest.mark.gpu
F32, F64 = torch.float32, torch.float64


def draws(seed):
    g = torch.Generator().manual_seed(seed)
    u = lambda a, b, *shape: a + (b - a) * torch.rand(*shape, generator=g, dtype=torch.float64)
    pick = lambda seq: seq[int(torch.randint(len(seq), (1,), generator=g))]
    return g, u, pick


def controller_spec(u, pick, dtype):
    rtol = 10.0 ** float(u(-6, -2.5, 1)) if dtype == F64 else 10.0 ** float(u(-5, -2.5, 1))
    ctrl = dict(kind=pick(["integral", "pid", "pid"]), atol=rtol * 10.0 ** float(u(-3, 0, 1)), rtol=rtol)
    if ctrl["kind"] == "pid":
        ctrl.update(pcoeff=float(u(0, 0.4, 1)), icoeff=float(u(0.3, 1.0, 1)), dcoeff=pick([0.0, float(u(0, 0.1, 1))]))
    return ctrl


def span_case(seed):
    """One of the three small systems on per-sample spans from t_start in -(0.5, 2) s to t_end in (0, 0.4) s (s = 1,
    0.01 or 37; partly backwards for the linear system), evaluation points sorted inside the span."""
    g, u, pick = draws(seed)
    dtype, B, E = pick([F32, F64]), int(torch.randint(1, 600, (1,), generator=g)), int(torch.randint(1, 40, (1,), generator=g))
    term = pick(["linear_decay", "vdp", "lorenz"])
    if term == "linear_decay":
        nf = int(torch.randint(1, 5, (1,), generator=g))
        f, y0 = to.LinearDecay(u(0.1, 3.0, B, nf).to(dtype)), u(-2, 2, B, nf)
    elif term == "vdp":
        f, y0 = to.VanDerPol(u(0.2, 8.0, B).to(dtype)), u(-2.5, 2.5, B, 2)
    else:
        f, y0 = to.Lorenz63(u(20.0, 35.0, B).to(dtype)), u(-10, 10, B, 3) + torch.tensor([0, 0, 20.0], dtype=torch.float64)
    back = (torch.rand(B, generator=g) < 0.4) & (term == "linear_decay")
    sign = torch.where(back, -1.0, 1.0).to(torch.float64)
    scale = pick([1.0, 1.0, 0.01, 37.0]) if term != "lorenz" else pick([1.0, 0.3])
    t_start, t_end = (-sign * u(0.5, 2.0, B) * scale).to(dtype), (sign * u(0.0, 0.4, B) * scale).to(dtype)
    t_eval = t_start[:, None] + (t_end - t_start)[:, None] * u(0, 1, B, E).sort(dim=1).values.to(dtype)
    if pick([True, False]):
        t_eval[:, 0] = t_start
    if pick([True, False]):
        t_eval[:, -1] = t_end
    lo, hi = torch.minimum(t_start, t_end)[:, None], torch.maximum(t_start, t_end)[:, None]
    t_eval = (torch.minimum(torch.maximum(t_eval, lo), hi) * sign[:, None].to(dtype)).cummax(dim=1).values * sign[:, None].to(dtype)
    ctrl, method = controller_spec(u, pick, dtype), pick(["dopri5", "tsit5"])
    kw = dict(t_start=t_start, t_end=t_end, max_steps=4000)
    if seed % 3 == 0:
        kw["dt0"] = (u(1e-3, 0.05, B) * sign * scale).to(dtype)
    return f, y0.to(dtype), t_eval, method, ctrl, kw


@pytest.mark.parametrize("seed", range(400, 440))
def test_spans_across_zero_through_every_whole_solve_dispatch(seed):
    f, y0, t_eval, method, ctrl, kw = span_case(seed)
    ref = c_oracle_solve(f, y0, t_eval, method, ctrl, **kw)
    for fast in (True, "one", "two", False):
        assert_identical(gpu_solve(f, y0, t_eval, method, ctrl, fast=fast, **kw), ref)


class OperatorTsit5(to.Tsit5):
    """A subclass is not recognised by the kernel paths: every protocol call runs as its own operator."""


class OperatorDopri5(to.Dopri5):
    pass


class OperatorHeun(to.Heun):
    pass


class OperatorEuler(to.Euler):
    pass


def same_bits(a, b, monotone=None):
    for key in ("n_steps", "n_accepted", "n_initialized", "n_f_evals"):
        assert torch.equal(a.stats[key], b.stats[key]), key
    assert torch.equal(a.status, b.status)
    written = torch.arange(a.ys.shape[1], device=a.ys.device)[None, :] < a.stats["n_initialized"][:, None]
    if monotone is not None:  # (n_initialized may count a row that never was written where the times go back and forth)
        written = written & monotone[:, None]
    x, y = a.ys[written], b.ys[written]
    assert bool(((x == y) | (x.isnan() & y.isnan())).all()), f"ys differ by up to {float((x - y).abs().nan_to_num().max()):.3e}"


def monotone_rows(problem):
    if problem.t_eval is None:
        return None
    d = (problem.t_eval[:, 1:] - problem.t_eval[:, :-1]) * torch.sign(problem.t_end - problem.t_start)[:, None]
    return (d >= 0).all(dim=1)


@pytest.mark.parametrize("seed", range(60))
def test_grid_and_mlp_kernels_against_the_protocol_path(seed):
    from test_large_rows_gpu import narrow_mlp_problem

    g, u, pick = draws(seed)
    u32 = lambda a, b, *shape: u(a, b, *shape).float()
    ctrl, method = controller_spec(u, pick, F32), pick(["tsit5", "dopri5"])
    B, E = int(torch.randint(1, 40, (1,), generator=g)), int(torch.randint(1, 30, (1,), generator=g))
    if seed % 2 == 0:
        n = pick([16, 32, 64, 128])
        f, y0, T1 = to.ReactionDiffusion(u32(0.001, pick([0.1, 1.0]), B).cuda(), n), u32(0, 1, B, n * n).cuda(), pick([0.5, 2.0, 8.0])
    else:
        w = narrow_mlp_problem(pick([64, 64, 32, 8, 3, 21]), pick([256, 100, 17]), B, seed=seed)
        f, y0, T1 = w.f, w.y0, pick([0.5, 1.0, 3.0])
    sign = torch.where((torch.rand(B, generator=g) < 0.3) & (T1 <= 1.0), -1.0, 1.0)
    t_start = u32(-1, 1, B) * pick([0.0, 1.0])
    t_end = t_start + sign * T1 * u32(0.3, 1.0, B)
    frac = u32(0, 1, B, E).sort(dim=1).values
    if pick([True, False]):
        frac[:, 0] = 0.0
    t_eval = ((t_start[:, None] + (t_end - t_start)[:, None] * frac) * sign[:, None]).cummax(dim=1).values * sign[:, None]
    if pick([True, False]):
        t_eval[:, -1] = t_end
    dt0 = pick([None, None, (u32(1e-3, 0.05, B) * sign).cuda()])
    if pick([False, False, False, True]):  # no evaluation points: the end point alone
        t_eval, E = None, 1
    problem = to.InitialValueProblem(y0, t_start.cuda(), t_end.cuda(), None if t_eval is None else t_eval.cuda())
    ours, other = {"tsit5": (to.Tsit5, OperatorTsit5), "dopri5": (to.Dopri5, OperatorDopri5)}[method]
    fused = to.AutoDiffAdjoint(ours(), make_controller(ctrl)).solve(problem, to.ODETerm(f), dt0=dt0)
    proto = to.AutoDiffAdjoint(other(), make_controller(ctrl)).solve(problem, to.ODETerm(f), dt0=dt0)
    if seed % 2 == 0:
        same_bits(fused, proto)
        return
    assert torch.equal(fused.status, proto.status)
    ok = fused.status == 0
    written = (torch.arange(E, device="cuda")[None, :] < torch.minimum(fused.stats["n_initialized"], proto.stats["n_initialized"])[:, None]) & ok[:, None]
    d = ((fused.ys - proto.ys).abs() / (1 + proto.ys.abs()))[written]
    assert d.numel() == 0 or float(d.max()) < 2e-2
    assert ((fused.stats["n_steps"] - proto.stats["n_steps"]).abs()[ok] <= 2 + proto.stats["n_steps"][ok] // 4).all()


def on_the_gpu(f, y0, t_start, t_end, t_eval, dt0, time_dtype, data_dtype):
    mv = lambda x, dt: None if x is None else x.to(dt).cuda()
    table = f.builtin_params().to(data_dtype)
    fd = type(f)(table if isinstance(f, to.LinearDecay) else table[:, 0]).cuda()
    return fd, to.InitialValueProblem(mv(y0, data_dtype), mv(t_start, time_dtype), mv(t_end, time_dtype), mv(t_eval, time_dtype)), mv(dt0, time_dtype)


@pytest.mark.parametrize("seed", range(900, 940))
def test_mixed_dtypes_general_kernel_against_the_per_step_kernels(seed):
    f, y0, t_eval, t_start, t_end, method, ctrl, max_steps, dt0 = wild_case(seed)
    if seed % 3 == 0:
        y0 = poisoned(y0, seed)
    time_dtype, data_dtype = (F64, F32) if seed % 2 else (F32, F64)
    fd, problem, dt0 = on_the_gpu(f, y0, t_start, t_end, t_eval, dt0, time_dtype, data_dtype)
    solver = lambda: to.AutoDiffAdjoint({"tsit5": to.Tsit5, "dopri5": to.Dopri5}[method](), make_controller(ctrl), max_steps=min(max_steps, 300))
    whole = solver().solve(problem, to.ODETerm(fd), dt0=dt0)
    stepwise = solver().solve(problem, to.ODETerm(lambda t, y: fd(t, y)), dt0=dt0)
    same_bits(whole, stepwise, monotone_rows(problem))


@pytest.mark.parametrize("seed", range(40))
def test_heun_and_euler_per_step_kernels_against_the_operator_path(seed):
    f, y0, t_eval, t_start, t_end, _, ctrl, max_steps, dt0 = wild_case(seed)
    g, u, pick = draws(seed)
    method, fixed = pick(["heun", "euler"]), pick([True, False])
    ctrl = dict(ctrl, rtol=max(ctrl["rtol"], 1e-3), atol=max(ctrl["atol"], 1e-5))
    if seed % 4 == 0:
        y0 = poisoned(y0, seed)
    time_dtype, data_dtype = pick([(F32, F32), (F64, F64), (F64, F32), (F32, F64)])
    if fixed or (method == "euler" and dt0 is None):  # (Euler under an adaptive controller keeps the step it starts with)
        dt0 = (t_end - t_start).double() / (30.0 + (torch.arange(y0.shape[0]) % 7) + 0.37)
    fd, problem, dt0 = on_the_gpu(f, y0, t_start, t_end, t_eval, dt0, time_dtype, data_dtype)
    controller = (lambda: to.FixedStepController()) if fixed else (lambda: make_controller(ctrl))
    opaque = lambda t, y: fd(t, y)
    kernels = to.AutoDiffAdjoint({"heun": to.Heun, "euler": to.Euler}[method](), controller(), max_steps=150).solve(problem, to.ODETerm(opaque), dt0=dt0)
    operators = to.AutoDiffAdjoint({"heun": OperatorHeun, "euler": OperatorEuler}[method](), controller(), max_steps=150).solve(problem, to.ODETerm(opaque), dt0=dt0)
    same_bits(kernels, operators, monotone_rows(problem))


def float64_draw_on_short_spans(seed):  # (not the spans scaled by 37: the linear system overflows there)
    _, y0, _, _, _, kw = span_case(seed)
    return y0.dtype == F64 and float(kw["t_start"].abs().max()) <= 3.0


@pytest.mark.parametrize("seed", [s for s in range(80000, 80100) if float64_draw_on_short_spans(s)][:24])
def test_one_kernel_reverse_sweep_against_the_sweep_in_torch_operations(seed):
    import torchode_amd.autodiff as autodiff

    f, y0, t_eval, method, ctrl, kw = span_case(seed)
    B = min(y0.shape[0], 64)
    cut = lambda x: None if x is None else x[:B].cuda()
    table = f.builtin_params()[:B].cuda()
    ctrl = dict(ctrl)
    kind = ctrl.pop("kind")
    for through in (True, False):
        results = {}
        for sweep in ("whole", "torch"):
            leaf = (table if isinstance(f, to.LinearDecay) else table[:, 0]).clone().requires_grad_()
            y = cut(y0).clone().requires_grad_()
            solver = to.AutoDiffAdjoint({"tsit5": to.Tsit5, "dopri5": to.Dopri5}[method](), to.PIDController(**ctrl) if kind == "pid" else to.IntegralController(**ctrl),
                                        backprop_through_step_size_control=through)  # fmt: skip
            solver.backward_whole_kernel, solver.backward_kernels = sweep == "whole", sweep != "torch"
            problem = to.InitialValueProblem(y, cut(kw["t_start"]), cut(kw["t_end"]), cut(t_eval))
            sol = solver.solve(problem, to.ODETerm(type(f)(leaf)), dt0=cut(kw.get("dt0")))
            if sweep == "whole":  # (again: the solver now knows the record's size and takes the recording whole-solve kernel)
                sol = solver.solve(problem, to.ODETerm(type(f)(leaf)), dt0=cut(kw.get("dt0")))
            E = t_eval.shape[1]
            written = (torch.arange(E, device="cuda")[None, :] < sol.stats["n_initialized"][:, None])[:, :, None]
            weights = torch.linspace(0.5, 1.5, E * y.shape[1], dtype=y.dtype, device="cuda").reshape(1, E, -1)
            loss = (torch.where(written, sol.ys, torch.zeros_like(sol.ys)) * weights).sum()
            results[sweep] = torch.autograd.grad(loss, [y, leaf], allow_unused=True), sol
            assert autodiff.LAST_SWEEP == sweep
        (got, a), (want, b) = results["whole"], results["torch"]
        assert torch.equal(a.status, b.status) and torch.equal(a.stats["n_steps"], b.stats["n_steps"])
        # (a sample whose last step is one unit in the last place long has a gradient through the step size rule that
        # is noise in every sweep: samples are compared where the torch sweep's own values are of ordinary size)
        for x, r in zip(got, want):
            if x is None or r is None:
                assert (x is None or not bool(x.any())) and (r is None or not bool(r.any()))
                continue
            ordinary = (r.abs().reshape(B, -1).amax(dim=1) < 1e4) & (b.status == 0)
            scale = r[ordinary].abs().max().clamp_min(1.0) if ordinary.any() else 1.0
            assert float(((x - r)[ordinary] / scale).abs().nan_to_num().max()) <= (1e-5 if through else 1e-8) if ordinary.any() else True
