"""GPU tests of ``torch.ops.torchode_amd``: the whole-solve entry point as an operator of PyTorch's
dispatcher (csrc/tode_torch_ops.cpp over tode_solve_builtin_auto), and ``torch.compile`` of
``AutoDiffAdjoint.solve`` capturing it as one node.  The eager solve of the same problem, which is
compared with the oracles elsewhere, is the checker: same kernels, so every bit must agree.
Reference: tests/torch_script_test.py (the compiled solver gives the eager solver's results)."""
import copy

import pytest
import torch

import torchode_amd as to
from torchode_amd import _lib, ops

pytestmark = pytest.mark.gpu
DEV = "cuda"


def same_solution(a, b):
    assert a.ys.dtype == b.ys.dtype and a.ys.shape == b.ys.shape
    # (a sample that stops early leaves the rest of its row unset, as in the reference: compare what was written)
    written = (torch.arange(a.ys.shape[1], device=a.ys.device)[None, :] < a.stats["n_initialized"][:, None])[:, :, None]
    assert bool(((a.ys == b.ys) | (a.ys.isnan() & b.ys.isnan()) | ~written).all())
    assert torch.equal(a.status, b.status) and torch.equal(a.ts, b.ts)
    assert set(a.stats) == set(b.stats)
    for key in a.stats:
        assert torch.equal(a.stats[key].cpu(), b.stats[key].cpu()), key
        assert a.stats[key].shape == b.stats[key].shape and a.stats[key].dtype == b.stats[key].dtype


def problem_of(name, batch, dtype, case="plain"):
    w = to.workloads.make(name, batch=batch, dtype=dtype)
    t_eval = w.t_eval.clone()
    dt0 = None
    if case == "non-monotone":
        t_eval[::5, 3], t_eval[::5, 7] = t_eval[::5, 7].clone(), t_eval[::5, 3].clone()
    if case == "dt0":
        dt0 = torch.full((batch,), 1e-3, dtype=dtype, device=DEV)
    y0 = w.y0.clone()
    if case == "non-finite":
        y0[3] = float("nan")
    if case == "end-only":
        return w, to.InitialValueProblem(y0.to(DEV), t_eval[:, 0].to(DEV), t_eval[:, -1].to(DEV)), dt0
    return w, to.InitialValueProblem(y0.to(DEV), t_eval=t_eval.to(DEV)), dt0


def solver_of(w, **kw):
    method = {"tsit5": to.Tsit5, "dopri5": to.Dopri5}[w.method]()
    c = dict(w.controller)
    kind = c.pop("kind")
    extra = {k: kw.pop(k) for k in ("dt_min", "dt_max") if k in kw}
    controller = to.PIDController(**c, **extra) if kind == "pid" else to.IntegralController(**c, **extra)
    return to.AutoDiffAdjoint(method, controller, **kw)


class Captured:
    """A compiler backend that runs the captured program as it is and keeps the names of its operator calls."""

    def __init__(self):
        self.calls = []

    def __call__(self, gm, example_inputs):
        self.calls.append([str(n.target) for n in gm.graph.nodes if n.op == "call_function"])
        return gm.forward


CASES = [
    ("vdp", 300, torch.float32, "plain", {}),
    ("vdp", 300, torch.float64, "plain", {}),
    ("lorenz", 200, torch.float32, "plain", {}),
    ("linear_decay", 100, torch.float64, "plain", {}),
    ("vdp", 200, torch.float32, "end-only", {}),
    ("vdp", 200, torch.float32, "dt0", {}),
    ("vdp", 200, torch.float32, "non-monotone", {}),  # general kernel, with the pending mask
    ("vdp", 200, torch.float32, "non-finite", {}),  # a non-success status: general kernel with an iteration cap
    ("vdp", 200, torch.float32, "plain", dict(max_steps=20)),
    ("lorenz", 200, torch.float64, "plain", dict(dt_max=0.01)),  # step size limits: general kernel only
    ("mlp", 64, torch.float32, "plain", {}),
    ("reaction_diffusion", 4, torch.float32, "plain", {}),
    ("reaction_diffusion", 3, torch.float64, "plain", {}),
    ("mlp", 64, torch.float32, "end-only", {}),
    ("reaction_diffusion", 4, torch.float32, "end-only", {}),
]


@pytest.mark.parametrize("name,batch,dtype,case,kw", CASES, ids=lambda v: str(v).replace("torch.", "") if not isinstance(v, dict) else "-".join(v) or "default")
def test_compiled_solve_is_one_operator_and_equals_the_eager_solve(name, batch, dtype, case, kw):
    torch._dynamo.reset()
    w, problem, dt0 = problem_of(name, batch, dtype, case)
    term = to.ODETerm(copy.deepcopy(w.f).to(DEV))
    solver = solver_of(w, **kw)
    with torch.no_grad():
        eager = solver.solve(problem, term, dt0=dt0)
        backend = Captured()
        compiled = torch.compile(solver.solve, backend=backend, fullgraph=True)
        traced = compiled(problem, term, dt0=dt0)
        again = compiled(problem, term, dt0=dt0)
    same_solution(traced, eager)
    same_solution(again, eager)
    assert len(backend.calls) == 1  # one program, captured once
    solves = [c for c in backend.calls[0] if c.startswith("torchode_amd.")]
    assert solves == (["torchode_amd.mlp_pack_weights", "torchode_amd.solve_builtin"] if name == "mlp" else ["torchode_amd.solve_builtin"])
    if case == "non-finite":
        assert (eager.status != 0).any()
    if kw.get("max_steps"):
        assert (eager.status == 3).any()


@pytest.mark.parametrize("time_dtype,data_dtype", [(torch.float64, torch.float32), (torch.float32, torch.float64)], ids=["t64-y32", "t32-y64"])
def test_compiled_solve_with_time_and_data_in_different_dtypes(time_dtype, data_dtype):
    torch._dynamo.reset()
    w = to.workloads.make("lorenz", batch=100, dtype=torch.float64)
    f = type(w.f)(w.f.builtin_params().to(data_dtype)[:, 0]).to(DEV)
    problem = to.InitialValueProblem(w.y0.to(data_dtype).to(DEV), t_eval=w.t_eval.to(time_dtype).to(DEV))
    term, solver = to.ODETerm(f), solver_of(w)
    with torch.no_grad():
        eager = solver.solve(problem, term)
        backend = Captured()
        traced = torch.compile(solver.solve, backend=backend, fullgraph=True)(problem, term)
    same_solution(traced, eager)
    assert traced.ys.dtype == data_dtype and traced.ts.dtype == time_dtype
    assert [c for c in backend.calls[0] if c.startswith("torchode_amd.")] == ["torchode_amd.solve_builtin"]


def test_operator_called_directly_and_its_tracing_rule():
    w, problem, _ = problem_of("vdp", 128, torch.float32)
    term = to.ODETerm(copy.deepcopy(w.f).to(DEV))
    solver = solver_of(w)
    with torch.no_grad():
        eager = solver.solve(problem, term)
    kind, control = solver.step_size_controller.control_values()
    args = (problem.y0, problem.t_start, problem.t_end, problem.t_eval, None, term.f.builtin_params(), None, solver.step_method.method_id,
            term.f.builtin_kind, [], kind, control, -1, True)  # fmt: skip
    ops.load()
    ys, n_steps, n_accepted, n_initialized, status, iterations = torch.ops.torchode_amd.solve_builtin(*args)
    assert torch.equal(ys, eager.ys) and torch.equal(n_steps, eager.stats["n_steps"]) and torch.equal(n_accepted, eager.stats["n_accepted"])
    assert torch.equal(n_initialized, eager.stats["n_initialized"]) and torch.equal(status, eager.status)
    assert iterations.device.type == "cpu" and 2 + 6 * int(iterations) == int(eager.stats["n_f_evals"][0])
    # schema, tracing rule (shapes, dtypes, devices of the results) and dispatch registrations, checked by PyTorch's own tool
    torch.library.opcheck(torch.ops.torchode_amd.solve_builtin, args, test_utils=("test_schema", "test_faketensor"))
    with pytest.raises(RuntimeError, match="controller kind"):
        torch.ops.torchode_amd.solve_builtin(*args[:10], 7, *args[11:])
    with pytest.raises(NotImplementedError):
        torch.ops.torchode_amd.solve_builtin(*(a.cpu() if isinstance(a, torch.Tensor) else a for a in args))


def test_a_solve_the_operator_does_not_cover_leaves_the_captured_program_and_runs_as_usual():
    torch._dynamo.reset()
    w, problem, _ = problem_of("vdp", 100, torch.float32)
    mu = w.f.mu.to(DEV)

    def rhs(t, y):  # a user's right-hand side: per-step kernels, nothing to capture
        x, v = y[:, 0], y[:, 1]
        return torch.stack((v, mu * (1 - x * x) * v - x), dim=1)

    solver = solver_of(w)
    with torch.no_grad():
        eager = solver.solve(problem, to.ODETerm(rhs))
        backend = Captured()
        traced = torch.compile(solver.solve, backend=backend)(problem, to.ODETerm(rhs))
    same_solution(traced, eager)
    assert not any(c.startswith("torchode_amd.") for calls in backend.calls for c in calls)


def test_gradients_are_not_silently_dropped_under_compile():
    torch._dynamo.reset()
    w, problem, _ = problem_of("vdp", 32, torch.float64)
    y0 = problem.y0.clone().requires_grad_()
    problem = to.InitialValueProblem(y0, t_eval=problem.t_eval)
    term = to.ODETerm(copy.deepcopy(w.f).to(DEV))
    solver = solver_of(w)
    sol = torch.compile(solver.solve)(problem, term)
    assert sol.ys.requires_grad  # left the captured program: the differentiable path ran
    (g,) = torch.autograd.grad(sol.ys[:, -1].sum(), y0)
    ref = solver.solve(problem, term)
    (g_ref,) = torch.autograd.grad(ref.ys[:, -1].sum(), y0)
    assert torch.allclose(g, g_ref, rtol=1e-9, atol=1e-11)
