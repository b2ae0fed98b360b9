#!/usr/bin/env python3
"""Benchmark of the batch-parallel adaptive RK solve loop on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]                 the headline + every other configuration
    python bench.py --workload vdp|lorenz|linear_decay|reaction_diffusion|mlp [--dtype f32|f64] [--path auto|per-step] ...
                                                                         one configuration alone (what the profiles run)

A "step" is one full solve of the workload's batch (start step, adaptive loop,
dense output, stats) with inputs resident in HBM.  Prints ONE JSON line.

* value        RK sample-steps per second (sum over samples of attempted steps / wall time) of the
               headline configuration, Van der Pol B = 65536 float32 Tsit5 + PID; `ivps_per_s` and
               `equiv_hbm_gbps` are the other two figures of the metric.
* roofline     dominant kernel = the persistent solve kernel.  `achieved` = algorithmic bytes
               of one launch (sum_b n_steps[b] * bytes_step + B * bytes_dense) divided by the
               kernel's average duration, measured with HIP events recorded around the kernel
               on the stream it is launched on.  The neural ODE is bounded by the matrix cores
               instead: algorithmic flops per launch over the same duration.
* cpu_baseline the same loop issued as ATen CPU operations (oracle/torch_loop.py, the closest
               stand-in for running the reference on the host) on the host cores this process
               may use, on a bounded prefix of the batch; `cpu_baseline_compiled` is the same
               function under torch.compile (what the reference's README recommends), its compile
               time reported and not counted; `cpu_baseline_scalar_c` is the scalar C oracle
               with OpenMP.  Reported baselines, not targets.
* configs      without --workload: the same measurement (value, roofline, cpu_baseline, ...) for
               each of the other configurations -- linear decay float64, Van der Pol float64,
               Lorenz, the neural ODE with float32 and with bfloat16 matrix-core inputs,
               reaction-diffusion -- each at its full size.  Compiled CPU legs are taken in this
               order while the run's time budget lasts; one that did not fit says so.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
MFMA_FP32_PEAK_TFLOPS = 157.3
MFMA_BF16_PEAK_TFLOPS = 2500.0
# HBM bytes per launch of the solve kernel, from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this script (the
# summaries under profiles/ name their commands).  A counter run is a run of its own, so these are constants read from
# those summaries, not something this run measures: the output says so (`traffic_source`), and a shape without a
# summary reports null.
TRAFFIC_PROFILES = {
    ("vdp", "torch.float32", 65536): "profiles/solve_pair_kernel_vdp_f32_b65536_hbm_traffic.txt",
    ("vdp", "torch.float64", 65536): "profiles/solve_pair_kernel_vdp_f64_b65536_hbm_traffic.txt",
    ("lorenz", "torch.float32", 1048576): "profiles/solve_fast_kernel_lorenz_f32_b1048576_hbm_traffic.txt",
    ("reaction_diffusion", "torch.float32", 512): "profiles/solve_grid_kernel_reaction_diffusion_f32_b512_hbm_traffic.txt",
    ("mlp", "torch.float32", 4096): "profiles/solve_mlp_kernel_mlp_f32_b4096_hbm_traffic.txt",
}
MEASURED_TRAFFIC_BYTES = {
    # profiles/solve_pair_kernel_vdp_f32_b65536_hbm_traffic.txt: (6871.2 KiB x 2.000 + 32926.0 KiB x 1.000) x 1024
    ("vdp", "torch.float32", 65536): 47.79e6,
    # profiles/solve_pair_kernel_vdp_f64_b65536_hbm_traffic.txt: (25316.5 KiB x 2.000 + 101408.5 KiB x 1.000) x 1024
    ("vdp", "torch.float64", 65536): 155.69e6,
    # profiles/solve_fast_kernel_lorenz_f32_b1048576_hbm_traffic.txt: (78276.2 KiB x 2.000 + 934960.1 KiB x 1.000) x 1024
    ("lorenz", "torch.float32", 1048576): 1117.71e6,
    # profiles/solve_grid_kernel_reaction_diffusion_f32_b512_hbm_traffic.txt: (4393 KiB x 2.000 + 819301 KiB x 1.000) x 1024
    ("reaction_diffusion", "torch.float32", 512): 847.96e6,
    # profiles/solve_mlp_kernel_mlp_f32_b4096_hbm_traffic.txt: (1504 KiB x 2.000 + 20624 KiB x 1.000) x 1024
    ("mlp", "torch.float32", 4096): 24.20e6,
}

# (workload, dtype flag, matrix-core inputs of the neural ODE) after the headline, in the order their compiled CPU legs are taken
OTHER_CONFIGS = [
    ("linear_decay", "f64", "float32"),
    ("vdp", "f64", "float32"),
    ("lorenz", "f32", "float32"),
    ("mlp", "f32", "float32"),
    ("reaction_diffusion", "f32", "float32"),
    ("mlp", "f32", "bfloat16"),
]
START = time.perf_counter()


def traffic_source(key):
    if key not in MEASURED_TRAFFIC_BYTES:
        return None
    return f"{TRAFFIC_PROFILES[key]}: rocprofv3 --pmc counter runs of this script, read from that summary, not measured in this run"


def measure(args, name, dtype_flag, mlp_inputs, steps, warmup, path=None, graph_iterations=-1, batch_copies=None):
    """One configuration on the GPU: wall time of `steps` solves, kernel time by HIP events, roofline."""
    path = args.path if path is None else path
    graph_iterations = args.graph_iterations if graph_iterations == -1 else graph_iterations
    import torch

    import torchode_amd as to
    from torchode_amd import _lib

    dtype = {None: None, "f32": torch.float32, "f64": torch.float64}[dtype_flag]
    w = to.workloads.make(name, batch=args.batch, dtype=dtype, device="cuda")
    dtype = w.y0.dtype
    if w.name == "mlp":
        w.f.matrix_inputs = mlp_inputs
    batch_copies = args.batch_copies if batch_copies is None else batch_copies
    if batch_copies > 1:  # (a larger batch of the same problems: for terms without per-sample parameters)
        assert w.name == "mlp", "--batch-copies is for the mlp workload (its weights are shared by the batch)"
        w = w._replace(y0=w.y0.repeat(batch_copies, 1).contiguous(), t_eval=w.t_eval.repeat(batch_copies, 1).contiguous())
    B, F = w.y0.shape
    E = w.t_eval.shape[1]
    spec = dict(w.controller)
    kind = spec.pop("kind")
    ctrl = to.PIDController(**spec) if kind == "pid" else to.IntegralController(**spec)
    solver = to.AutoDiffAdjoint(to.Tsit5() if w.method == "tsit5" else to.Dopri5(), ctrl, graph_iterations=graph_iterations)
    problem = to.InitialValueProblem(w.y0, t_eval=w.t_eval)
    term = to.ODETerm(w.f if path == "auto" else (lambda t, y, f=w.f: f(t, y)))

    with torch.no_grad():  # a forward solve: nothing here asks for gradients
        for _ in range(warmup):
            sol = solver.solve(problem, term)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            sol = solver.solve(problem, term)
        torch.cuda.synchronize()
        wall = (time.perf_counter() - t0) / steps

        assert (sol.status == 0).all(), "benchmark solve did not succeed"
        sample_steps = int(sol.stats["n_steps"].sum().item())
        algo_bytes = sample_steps * w.bytes_step + B * w.bytes_dense

        # kernel-only duration: HIP events recorded by the library around the solve kernel
        _lib.set_kernel_timing(True)
        kms = []
        try:
            for _ in range(max(5, min(steps, 20))):
                solver.solve(problem, term)
                kms.append(_lib.last_solve_kernel_ms())
            kernel_name = _lib.last_solve_kernel_name()
            kernel_s = sum(kms) / len(kms) / 1e3
        except RuntimeError:
            # no whole-solve kernel for this workload: the solve is a sequence of per-call kernels
            # around the torch right-hand side, and the figure below is over the whole solve
            per_step = path == "per-step"
            kernel_name = ("per-step kernels" if per_step else "protocol path (one kernel per protocol call)") + " + torch right-hand side"
            if per_step and graph_iterations:
                kernel_name += f", {graph_iterations} iterations per HIP graph replay"
            kernel_s = wall
        _lib.set_kernel_timing(False)
    achieved = algo_bytes / kernel_s / 1e9
    roofline = {
        "bound": "hbm",
        "kernel": kernel_name,
        "achieved": achieved,
        "peak": HBM_PEAK_GBPS,
        "unit": "GB/s",
        "frac": achieved / HBM_PEAK_GBPS,
        # (the counter runs profiled the whole-solve kernel: nothing to quote for the per-step or the protocol path)
        "traffic": MEASURED_TRAFFIC_BYTES.get((w.name, str(dtype), B)) if kernel_name.startswith("tode::solve") else None,
        "traffic_source": traffic_source((w.name, str(dtype), B)) if kernel_name.startswith("tode::solve") else None,
        "algorithmic_bytes_per_launch": algo_bytes,
        "bytes_per_sample_step": w.bytes_step,
        "bytes_dense_per_sample": w.bytes_dense,
        "kernel_ms": kernel_s * 1e3,
    }
    if path == "per-step":
        # with an external f the stages go through HBM: per sample-step the stage kernels read 27 and
        # write 6 rows, f reads and writes a row six times, the finishing kernel reads 9 and writes 2
        sd = w.y0.element_size()
        roofline["own_compulsory_bytes_per_launch"] = sample_steps * (56 * F * sd + w.bytes_step - 4 * F * sd)
    if w.name == "mlp":
        # dense contractions: the matrix cores bound this workload, not HBM.  Per evaluation of f and
        # sample 2*(65*256 + 256*64) flops; a sample evaluates f twice for the first step size and six
        # times per step; about 5000 flops per step for the Runge-Kutta sums, error norm and control.
        H, Fin = w.f.W1.shape
        flops_f = 2 * (Fin * H + H * F)
        flops = (2 * B + 6 * sample_steps) * flops_f + 5000 * sample_steps
        tflops = flops / kernel_s / 1e12
        peak = MFMA_FP32_PEAK_TFLOPS if mlp_inputs == "float32" else MFMA_BF16_PEAK_TFLOPS
        roofline = {
            "bound": "mfma",
            "kernel": kernel_name,
            "achieved": tflops,
            "peak": peak,
            "unit": "TFLOP/s",
            "frac": tflops / peak,
            "traffic": MEASURED_TRAFFIC_BYTES.get((w.name, str(dtype), B)) if mlp_inputs == "float32" else None,
            "traffic_source": traffic_source((w.name, str(dtype), B)) if mlp_inputs == "float32" else None,
            "algorithmic_flops_per_launch": flops,
            "flops_per_rhs_evaluation_per_sample": flops_f,
            "kernel_ms": kernel_s * 1e3,
        }
    result = {
        "value": sample_steps / wall,
        "unit": "sample-steps/s",
        "steps": steps,
        "warmup": warmup,
        "ms_per_step": wall * 1e3,
        "dtype": {torch.float32: "f32", torch.float64: "f64"}[dtype] + (" (bf16 matrix-core inputs)" if w.name == "mlp" and mlp_inputs == "bfloat16" else ""),
        "config": {
            "workload": f"{w.name} B={B} F={F} E={E} {w.method}+{kind}",
            "controller": w.controller,
            "sample_steps_per_solve": sample_steps,
            "max_steps_per_sample": int(sol.stats["n_steps"].max().item()),
        },
        "ivps_per_s": B / wall,
        "equiv_hbm_gbps": algo_bytes / wall / 1e9,
        "roofline": roofline,
    }
    del sol, problem, w
    torch.cuda.empty_cache()
    return result


def measure_gradient(args, steps=10, warmup=3):
    """A differentiable solve of the headline configuration (Van der Pol float32, y0 and mu requiring grad) and the
    backward pass of sum(ys): the record of the loop state from the general whole-solve kernel, the reverse sweep in
    one kernel."""
    import torch

    import torchode_amd as to
    from torchode_amd import autodiff

    w = to.workloads.make("vdp", batch=args.batch, dtype=torch.float32, device="cuda")
    mu = w.f.builtin_params()[:, 0].clone().requires_grad_()
    y0 = w.y0.clone().requires_grad_()
    spec = dict(w.controller)
    spec.pop("kind")
    solver = to.AutoDiffAdjoint(to.Tsit5(), to.PIDController(**spec))
    problem, term = to.InitialValueProblem(y0, t_eval=w.t_eval), to.ODETerm(to.VanDerPol(mu))
    forward = backward = 0.0
    for i in range(warmup + steps):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        sol = solver.solve(problem, term)
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        grads = torch.autograd.grad(sol.ys.sum(), (y0, mu))
        torch.cuda.synchronize()
        t2 = time.perf_counter()
        if i >= warmup:
            forward, backward = forward + (t1 - t0), backward + (t2 - t1)
    assert all(bool(g.isfinite().all()) for g in grads)
    sample_steps = int(sol.stats["n_steps"].sum().item())
    return {
        "config": {"workload": f"vdp B={y0.shape[0]} F=2 E={w.t_eval.shape[1]} tsit5+pid, gradient of sum(ys) with respect to y0 and mu"},
        "forward_ms": forward / steps * 1e3,
        "backward_ms": backward / steps * 1e3,
        "reverse_sweep": autodiff.LAST_SWEEP,
        "value": sample_steps / ((forward + backward) / steps),
        "unit": "sample-steps/s (forward and backward)",
        "steps": steps,
        "warmup": warmup,
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default=None, choices=[None, "vdp", "lorenz", "linear_decay", "reaction_diffusion", "mlp"],
                    help="measure this configuration alone (default: the headline, Van der Pol float32, and then every other one under 'configs')")  # fmt: skip
    ap.add_argument("--dtype", default=None, choices=[None, "f32", "f64"])
    ap.add_argument("--batch", type=int, default=None, help="prefix of the workload's batch (default: full size)")
    ap.add_argument("--batch-copies", type=int, default=1, help="mlp workload: solve this many copies of the batch at once (B = 4096 x copies), to see the kernel with more than one workgroup per compute unit")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-compiled-baseline", action="store_true", help="skip the torch.compile CPU legs (about a minute of compilation each)")
    ap.add_argument(
        "--path",
        default="auto",
        choices=["auto", "per-step"],
        help="per-step: hide the built-in term behind a plain callable, so that the solve runs through the per-step kernels around the torch right-hand side, as for any user-defined f",
    )
    ap.add_argument("--mlp-inputs", default="float32", choices=["float32", "bfloat16"], help="mlp workload: what the matrix cores take as inputs (bfloat16: a reduced-precision variant, reported against the bf16 peak)")
    ap.add_argument("--gradient", action="store_true", help="measure the differentiable solve of the headline configuration alone (forward with its record, backward)")
    ap.add_argument("--graph-iterations", type=int, default=None, help="per-step path: replay this many iterations at a time from a HIP graph")
    ap.add_argument("--cpu-baseline-seconds", type=float, default=10.0, help="CPU work the headline's eager baseline is sized to (the other configurations take 0.4 of it)")
    ap.add_argument("--time-budget", type=float, default=420.0, help="seconds the whole run aims to stay within: a compiled CPU leg is started only while 100 s of it are left")
    ap.add_argument(
        "--calibration-copy-mib",
        type=int,
        default=0,
        help="also run one plain device copy of this many MiB (a known-size reference for scaling rocprofv3's FETCH_SIZE / WRITE_SIZE counters)",
    )
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU; --gpus must be 1 (with more GPUs the batch axis would be split, every GPU solving its own samples)")

    import torch

    assert torch.cuda.is_available(), "bench.py needs a GPU"

    if args.calibration_copy_mib:
        src = torch.ones(args.calibration_copy_mib * 2**20 // 4, dtype=torch.float32, device="cuda")
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        dst.copy_(src)  # reads and writes exactly calibration_copy_mib MiB
        torch.cuda.synchronize()
        del src, dst

    if args.gradient:
        print(json.dumps(measure_gradient(args, steps=args.steps if args.steps != 50 else 10)))
        return
    everything = args.workload is None
    head = ("vdp", "f32", "float32") if everything else (args.workload, args.dtype, args.mlp_inputs)
    result = measure(args, *head, args.steps, args.warmup)
    out = {
        "metric": "RK sample-steps/s (adaptive Tsit5/Dopri5 solve, whole batch)",
        "value": result.pop("value"),
        "unit": result.pop("unit"),
        "n_gpus": 1,
        "steps": result.pop("steps"),
        "warmup": result.pop("warmup"),
        "ms_per_step": result.pop("ms_per_step"),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": result.pop("dtype"),
        "data": "synthetic",
        **result,
    }
    others = []
    if everything:
        for name, dtype_flag, mlp_inputs in OTHER_CONFIGS:
            others.append(measure(args, name, dtype_flag, mlp_inputs, max(5, args.steps // 2), max(2, args.warmup // 2)))

    if not args.no_cpu_baseline:
        # eager legs of every configuration first (seconds each), then the compiled legs while the budget lasts
        plans = [(out, *head, args.cpu_baseline_seconds)] + [(o, *c, 0.4 * args.cpu_baseline_seconds) for o, c in zip(others, OTHER_CONFIGS)]
        for entry, name, dtype_flag, mlp_inputs, seconds in plans:
            entry.update(cpu_baselines(args, name, dtype_flag, mlp_inputs, seconds))
        for entry, name, dtype_flag, mlp_inputs, seconds in plans:
            if args.no_compiled_baseline:
                entry["cpu_baseline_compiled"] = {"skipped": "--no-compiled-baseline"}
            elif args.time_budget - (time.perf_counter() - START) < 100.0:
                entry["cpu_baseline_compiled"] = {"skipped": f"the run's time budget of {args.time_budget:.0f} s leaves no room for another compilation (about a minute each)"}
            else:
                entry["cpu_baseline_compiled"] = compiled_baseline(args, name, dtype_flag, mlp_inputs, entry["cpu_baseline"])
    if everything:
        out["configs"] = others
        # the headline configuration with its right-hand side hidden behind a plain callable, as any user-defined f is:
        # the per-step kernels around torch's evaluation of f, eager and with iterations replayed from a HIP graph
        out["user_defined_f"] = [
            measure(args, "vdp", "f32", "float32", 5, 2, path="per-step", graph_iterations=None),
            measure(args, "vdp", "f32", "float32", 5, 2, path="per-step", graph_iterations=2),
        ]
        out["gradient"] = measure_gradient(args)
        # the neural ODE at sixteen times its batch (not a BASELINE configuration): two workgroups per compute unit
        # fill each other's waits for barriers and LDS, which the one workgroup per compute unit of B=4096 cannot
        out["larger_batch"] = [measure(args, "mlp", "f32", "float32", 10, 2, batch_copies=16)]
    out["bench_seconds"] = time.perf_counter() - START
    print(json.dumps(out))


def host_threads():
    """Threads the CPU legs use: torch's default, which follows OMP_NUM_THREADS / the cores this process may use."""
    import torch

    return torch.get_num_threads()


def cpu_workload(name, dtype_flag, mlp_inputs, batch):
    import torch

    import torchode_amd as to

    dtype = {None: None, "f32": torch.float32, "f64": torch.float64}[dtype_flag]
    w = to.workloads.make(name, batch=batch, dtype=dtype)
    if name == "mlp":
        w.f.matrix_inputs = mlp_inputs
    return w


def cpu_baselines(args, name, dtype_flag, mlp_inputs, seconds):
    """Host-core baselines on a bounded prefix of the same workload."""
    import torch

    from oracle import c_oracle, torch_loop

    cores = host_threads()
    full = cpu_workload(name, dtype_flag, mlp_inputs, args.batch)
    B = full.y0.shape[0]
    ww = cpu_workload(name, dtype_flag, mlp_inputs, min(B, {"reaction_diffusion": 8, "mlp": 256}.get(name, 2048)))
    ctrl = torch_loop.Controller(**ww.controller)
    torch_loop.solve(ww.f, ww.y0, ww.t_eval, method=ww.method, controller=ctrl)  # warm up
    t0 = time.perf_counter()
    torch_loop.solve(ww.f, ww.y0, ww.t_eval, method=ww.method, controller=ctrl)
    per_sample = (time.perf_counter() - t0) / ww.y0.shape[0]
    # the loop's cost per iteration has a fixed part, so small batches overestimate the cost per
    # sample: the sample below is sized generously and the time actually taken is reported
    n = int(min(B, max(ww.y0.shape[0], 2 * seconds / per_sample)))
    wc = cpu_workload(name, dtype_flag, mlp_inputs, n)
    t_torch, steps_n, solves = 0.0, 0, 0
    while solves == 0 or (t_torch < 0.8 * seconds and solves < 64):  # whole workload too short: repeat it
        t0 = time.perf_counter()
        ref = torch_loop.solve(wc.f, wc.y0, wc.t_eval, method=wc.method, controller=ctrl)
        t_torch += time.perf_counter() - t0
        steps_n += int(ref["n_steps"].sum())
        solves += 1

    first = {
        "cpu_baseline": {
            "value": steps_n / t_torch,
            "unit": "sample-steps/s",
            "cores": cores,
            "host_cpu_count": os.cpu_count(),
            "kind": "port",
            "sample": f"first {n} of {B} samples of the workload, {solves} eager solve(s) of the ATen-op restatement (torch {torch.__version__})",
            "sample_batch": n,
            "seconds": t_torch,
        }
    }
    if name not in c_oracle.TERMS:
        return first
    nc = min(B, 262144)
    wc2 = cpu_workload(name, dtype_flag, mlp_inputs, nc)
    cfg = c_oracle.make_config(method=wc2.method, term=name, nthreads=cores, **wc2.controller)
    c_oracle.solve(cfg, ww.f.builtin_params(), ww.y0, ww.t_eval)
    t0 = time.perf_counter()
    refc = c_oracle.solve(cfg, wc2.f.builtin_params(), wc2.y0, wc2.t_eval)
    t_c = time.perf_counter() - t0
    return {
        **first,
        "cpu_baseline_scalar_c": {
            "value": int(refc["n_steps"].sum()) / t_c,
            "unit": "sample-steps/s",
            "cores": cores,
            "kind": "port",
            "sample": f"first {nc} of {B} samples, one solve of the scalar C oracle (OpenMP over samples)",
            "seconds": t_c,
        },
    }


def compiled_baseline(args, name, dtype_flag, mlp_inputs, eager):
    """The eager leg's function under torch.compile, on the eager leg's sample.  The reference recommends compiling
    the solver (its README; its loop has a data-dependent end, so the compiled function is a chain of graphs with a
    break per iteration).  Compilation happens in the first call and is reported, not counted.  A host on which the
    compiler cannot run gives {"error": first line of the failure}."""
    import torch

    from oracle import torch_loop

    wc = cpu_workload(name, dtype_flag, mlp_inputs, eager["sample_batch"])
    ctrl = torch_loop.Controller(**wc.controller)

    def run(f, y0, t_eval):
        return torch_loop.solve(f, y0, t_eval, method=wc.method, controller=ctrl)

    try:
        import torch._dynamo

        torch._dynamo.reset()
        torch._dynamo.config.cache_size_limit = 64
        compiled = torch.compile(run)
        t0 = time.perf_counter()
        out = compiled(wc.f, wc.y0, wc.t_eval)
        t_compile = time.perf_counter() - t0
        want = max(1.0, min(eager["seconds"], 6.0))
        t_run, steps_n, solves = 0.0, 0, 0
        while solves == 0 or (t_run < want and solves < 64):
            t0 = time.perf_counter()
            out = compiled(wc.f, wc.y0, wc.t_eval)
            t_run += time.perf_counter() - t0
            steps_n += int(out["n_steps"].sum())
            solves += 1
    except Exception as e:  # noqa: BLE001 -- whatever the compiler stack raises on this host is the result
        text = str(e).strip().splitlines()
        return {"error": f"{type(e).__name__}: {text[0][:300] if text else ''}"}
    return {
        "value": steps_n / t_run,
        "unit": "sample-steps/s",
        "cores": eager["cores"],
        "kind": "port",
        "sample": f"first {eager['sample_batch']} samples of the workload, {solves} solve(s) of torch.compile(the ATen-op restatement) after a first call of {t_compile:.0f} s that compiled it",
        "seconds": t_run,
        "compile_seconds": t_compile,
        "speedup_over_eager": (steps_n / t_run) / eager["value"],
    }


if __name__ == "__main__":
    main()
