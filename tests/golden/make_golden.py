"""Writes tests/golden/*.json: golden vectors of the solve loop on the seeded workloads.

    python tests/golden/make_golden.py

Source of the vectors: oracle/torch_loop.py -- the reference's loop issued operation by
operation as ATen CPU calls -- run in the authoring container (torch 2.10.0+rocm7.0, CPU
capability AVX512, Intel MKL, opt_einsum absent, 8 threads).  ATen's results depend on the
host (MKL picks other kernels on other CPUs, vectorised and scalar tails round differently),
which is why the vectors are committed instead of being recomputed where the tests run.  The
script refuses to write a fixture unless the scalar C oracle (oracle/erk_oracle.c) reproduces
the ATen result bit for bit, so each file pins both.  The reference package itself could not
be imported here (its torchtyping dependency is absent); these are vectors of its restatement.
Inputs are identified by sha256, outputs are the per-sample integer stats (or their
sha256 for the large cases), the sha256 of ys and the exact ys of a strided subset.
"""
import hashlib
import json
import os
import sys

import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

import torchode_amd as to  # noqa: E402
from oracle import c_oracle, torch_loop  # noqa: E402

CASES = [
    ("linear_decay", 256, torch.float64),
    ("linear_decay", 256, torch.float32),
    ("vdp", 1024, torch.float32),
    ("vdp", 1024, torch.float64),
    ("lorenz", 512, torch.float32),
    ("lorenz", 512, torch.float64),
    # full-size headline configuration and a large Lorenz prefix: digests only
    ("vdp", 65536, torch.float32),
    ("lorenz", 65536, torch.float32),
]
DIGEST_ABOVE = 4096  # larger cases store sha256 digests instead of the per-sample lists

# Workloads with long rows: vectors of the ATen-op oracle only (no scalar C restatement: ATen's
# order of summation in a 4096-element norm and in its matrix products is a property of its CPU
# build), to be compared at the floating point tolerance, not bit for bit.
TOLERANCE_CASES = [("reaction_diffusion", 16, torch.float32), ("mlp", 128, torch.float32)]


def sha(t: torch.Tensor) -> str:
    return hashlib.sha256(t.contiguous().numpy().tobytes()).hexdigest()


def hexlist(t: torch.Tensor):
    """Exact float values as hex strings (float.hex round-trips through float.fromhex)."""
    return [float(v).hex() for v in t.flatten().tolist()]


def make(name, batch, dtype):
    w = to.workloads.make(name, batch=batch, dtype=dtype)
    out = torch_loop.solve(w.f, w.y0, w.t_eval, method=w.method, controller=torch_loop.Controller(**w.controller))
    cfg = c_oracle.make_config(method=w.method, term=name, nthreads=4, **w.controller)
    chk = c_oracle.solve(cfg, w.f.builtin_params(), w.y0, w.t_eval)
    for key in ("ys", "n_steps", "n_accepted", "n_initialized", "status", "n_f_evals"):
        assert torch.equal(out[key], chk[key]), f"{name} {dtype}: C oracle and ATen-op oracle disagree on {key}"
    ys = out["ys"].double()
    sub = list(range(0, batch, max(1, batch // 16)))[:16]
    return {
        "source": f"oracle/torch_loop.py (ATen CPU ops), torch {torch.__version__}, {torch.backends.cpu.get_cpu_capability()}, "
        f"opt_einsum {torch.backends.opt_einsum.is_available()}; reproduced bit for bit by oracle/erk_oracle.c",
        "workload": name,
        "batch": batch,
        "dtype": str(dtype).replace("torch.", ""),
        "method": w.method,
        "controller": w.controller,
        "inputs_sha256": {"y0": sha(w.y0), "t_eval": sha(w.t_eval), "params": sha(w.f.builtin_params())},
        "n_f_evals": int(out["n_f_evals"][0]),
        **{
            key: (out[key].tolist() if batch <= DIGEST_ABOVE else {"sha256_int64": sha(out[key]), "sum": int(out[key].sum())})
            for key in ("n_steps", "n_accepted", "n_initialized", "status")
        },
        "ys_sha256": sha(out["ys"]),
        "ys_max_abs": float(ys.abs().max()).hex(),
        "subset": sub,
        "ys_subset": hexlist(out["ys"][sub]),
    }


# Time and data in different dtypes (reference problems.py:44-56): vectors of the ATen-op oracle alone (the scalar C
# oracle is written for one dtype); the per-step kernels and the operator path are compared with them bit for bit.
MIXED_CASES = [
    ("vdp", 512, torch.float64, torch.float32),
    ("vdp", 512, torch.float32, torch.float64),
    ("lorenz", 256, torch.float64, torch.float32),
    ("lorenz", 256, torch.float32, torch.float64),
]


def mixed_inputs(name, batch, time_dtype, data_dtype):
    """The float64 workload with its times rounded to one dtype and its state and parameters to the other."""
    w = to.workloads.make(name, batch=batch, dtype=torch.float64)
    params = w.f.builtin_params().to(data_dtype)
    f = type(w.f)(params[:, 0] if params.shape[1] == 1 else params)
    return w, f, w.y0.to(data_dtype), w.t_eval.to(time_dtype)


def make_mixed(name, batch, time_dtype, data_dtype):
    w, f, y0, t_eval = mixed_inputs(name, batch, time_dtype, data_dtype)
    out = torch_loop.solve(f, y0, t_eval, method=w.method, controller=torch_loop.Controller(**w.controller))
    assert out["ys"].dtype == data_dtype and (out["status"] == 0).all()
    sub = list(range(0, batch, max(1, batch // 16)))[:16]
    return {
        "source": f"oracle/torch_loop.py (ATen CPU ops), torch {torch.__version__}, {torch.backends.cpu.get_cpu_capability()}, "
        f"opt_einsum {torch.backends.opt_einsum.is_available()}; time and data dtypes differ",
        "workload": name,
        "batch": batch,
        "time_dtype": str(time_dtype).replace("torch.", ""),
        "data_dtype": str(data_dtype).replace("torch.", ""),
        "method": w.method,
        "controller": w.controller,
        "inputs_sha256": {"y0": sha(y0), "t_eval": sha(t_eval), "params": sha(f.builtin_params())},
        "n_f_evals": int(out["n_f_evals"][0]),
        **{key: out[key].tolist() for key in ("n_steps", "n_accepted", "n_initialized", "status")},
        "ys_sha256": sha(out["ys"]),
        "subset": sub,
        "ys_subset": hexlist(out["ys"][sub]),
    }


# Fixed steps (reference step_size_controllers.py:116-167) with Dopri5 / Tsit5: vectors of the ATen-op oracle alone.
FIXED_CASES = [("vdp", 256, torch.float32, "tsit5"), ("lorenz", 256, torch.float64, "dopri5")]


def fixed_inputs(name, batch, dtype):
    """The workload with a per-sample fixed step: the span cut into 60.37 to 66.37 parts (the last step is cut short)."""
    w = to.workloads.make(name, batch=batch, dtype=dtype)
    span = (w.t_eval[:, -1] - w.t_eval[:, 0]).double()
    dt0 = (span / (60.37 + torch.arange(batch, dtype=torch.float64) % 7)).to(dtype)
    return w, dt0


def make_fixed(name, batch, dtype, method):
    w, dt0 = fixed_inputs(name, batch, dtype)
    out = torch_loop.solve(w.f, w.y0, w.t_eval, method=method, controller=torch_loop.Controller("fixed", 0.0, 0.0), dt0=dt0)
    assert (out["status"] == 0).all() and torch.equal(out["n_steps"], out["n_accepted"]) and 61 <= int(out["n_steps"].min())
    sub = list(range(0, batch, max(1, batch // 16)))[:16]
    return {
        "source": f"oracle/torch_loop.py (ATen CPU ops), torch {torch.__version__}, {torch.backends.cpu.get_cpu_capability()}, "
        f"opt_einsum {torch.backends.opt_einsum.is_available()}; fixed steps",
        "workload": name,
        "batch": batch,
        "dtype": str(dtype).replace("torch.", ""),
        "method": method,
        "inputs_sha256": {"y0": sha(w.y0), "t_eval": sha(w.t_eval), "params": sha(w.f.builtin_params()), "dt0": sha(dt0)},
        "n_f_evals": int(out["n_f_evals"][0]),
        **{key: out[key].tolist() for key in ("n_steps", "n_accepted", "n_initialized", "status")},
        # (some of the stiffer Van der Pol samples blow up at these step sizes: NaN hashed as 0, its bits are not pinned)
        "ys_sha256_nan_as_zero": sha(out["ys"].nan_to_num(nan=0.0, posinf=float("inf"), neginf=float("-inf"))),
        "ys_finite_fraction": float(out["ys"].isfinite().double().mean()),
        "subset": sub,
        "ys_subset": hexlist(out["ys"][sub]),
    }


# Heun and Euler (reference heun.py, euler.py) with the three controllers: vectors of the ATen-op oracle alone.
#   (workload, batch, dtype, method, controller or None for the workload's own, parts of the span as the first step or None)
# (Without a first step the reference takes ``x ** (1 / order)`` in its choice of one, which for Heun's order 2 is ATen's
# square root kernel; that one comes from a vector math library on this host and is not the correctly rounded root for
# some 0.7 % of arguments.  Such a case is written as a tolerance-level vector: "bit_exact" false.)
LOW_ORDER_CASES = [
    ("vdp", 256, torch.float32, "heun", None, 400.37),
    ("lorenz", 256, torch.float64, "heun", dict(kind="integral", atol=1e-6, rtol=1e-4), 500.37),
    ("linear_decay", 256, torch.float64, "heun", dict(kind="integral", atol=1e-6, rtol=1e-4), None),
    ("linear_decay", 256, torch.float64, "heun", dict(kind="fixed", atol=0.0, rtol=0.0), 80.37),
    ("vdp", 256, torch.float32, "euler", dict(kind="fixed", atol=0.0, rtol=0.0), 200.37),
    ("linear_decay", 256, torch.float64, "euler", dict(kind="integral", atol=1e-6, rtol=1e-4), 300.37),
]


def low_order_inputs(name, batch, dtype, parts):
    w = to.workloads.make(name, batch=batch, dtype=dtype)
    if parts is None:
        return w, None
    span = (w.t_eval[:, -1] - w.t_eval[:, 0]).double()
    return w, (span / (parts + torch.arange(batch, dtype=torch.float64) % 7)).to(dtype)


def make_low_order(name, batch, dtype, method, controller, parts):
    w, dt0 = low_order_inputs(name, batch, dtype, parts)
    controller = dict(w.controller) if controller is None else controller
    out = torch_loop.solve_low_order(w.f, w.y0, w.t_eval, method=method, controller=torch_loop.Controller(**controller), dt0=dt0)
    assert (out["status"] == 0).all() and (out["n_initialized"] == w.t_eval.shape[1]).all()
    sub = list(range(0, batch, max(1, batch // 16)))[:16]
    return {
        "source": f"oracle/torch_loop.py::solve_low_order (ATen CPU ops), torch {torch.__version__}, {torch.backends.cpu.get_cpu_capability()}, "
        f"opt_einsum {torch.backends.opt_einsum.is_available()}",
        "workload": name,
        "batch": batch,
        "dtype": str(dtype).replace("torch.", ""),
        "method": method,
        "controller": controller,
        "first_step_parts": parts,
        "bit_exact": parts is not None,
        "inputs_sha256": {"y0": sha(w.y0), "t_eval": sha(w.t_eval), "params": sha(w.f.builtin_params())},
        "n_f_evals": int(out["n_f_evals"][0]),
        **{key: out[key].tolist() for key in ("n_steps", "n_accepted", "n_initialized", "status")},
        "ys_sha256_nan_as_zero": sha(out["ys"].nan_to_num(nan=0.0, posinf=float("inf"), neginf=float("-inf"))),
        "ys_finite_fraction": float(out["ys"].isfinite().double().mean()),
        "subset": sub,
        "ys_subset": hexlist(out["ys"][sub]),
    }


# Solves without evaluation points that stop early on max_steps (reference adjoints.py:176-181, 296-311): the one value
# returned per sample is the last step's interpolant evaluated at t_end, far outside the step (theta >> 1), which
# amplifies the last place of the dense-output weights by many orders of magnitude.  The case that tells the
# reference's Tsit5 weights (a sympy float expansion, tsit5.py:11-50) from an exact expansion of the same polynomials.
#   (workload, batch, dtype, max_steps)
EARLY_STOP_CASES = [("vdp", 256, torch.float64, 20), ("vdp", 256, torch.float32, 12)]


def early_stop_inputs(name, batch, dtype):
    w = to.workloads.make(name, batch=batch, dtype=dtype)
    return w, w.t_eval[:, 0].clone(), w.t_eval[:, -1].clone()


def make_early_stop(name, batch, dtype, max_steps):
    w, t_start, t_end = early_stop_inputs(name, batch, dtype)
    ctrl = torch_loop.Controller(**w.controller)
    out = torch_loop.solve(w.f, w.y0, None, method=w.method, controller=ctrl, t_start=t_start, t_end=t_end, max_steps=max_steps)
    cfg = c_oracle.make_config(method=w.method, term=name, nthreads=4, max_steps=max_steps, **w.controller)
    chk = c_oracle.solve(cfg, w.f.builtin_params(), w.y0, None, t_start=t_start, t_end=t_end)
    for key in ("ys", "n_steps", "n_accepted", "n_initialized", "status", "n_f_evals"):
        assert torch.equal(out[key], chk[key]), f"{name} {dtype}: C oracle and ATen-op oracle disagree on {key}"
    assert out["ys"].shape == (batch, 1, w.y0.shape[1]) and (out["status"] == 3).all() and (out["n_steps"] == max_steps).all()
    return {
        "source": f"oracle/torch_loop.py (ATen CPU ops), torch {torch.__version__}, {torch.backends.cpu.get_cpu_capability()}, "
        f"opt_einsum {torch.backends.opt_einsum.is_available()}; reproduced bit for bit by oracle/erk_oracle.c; no evaluation points, "
        "every sample stopped by max_steps",
        "workload": name,
        "batch": batch,
        "dtype": str(dtype).replace("torch.", ""),
        "method": w.method,
        "controller": w.controller,
        "max_steps": max_steps,
        "inputs_sha256": {"y0": sha(w.y0), "t_start": sha(t_start), "t_end": sha(t_end), "params": sha(w.f.builtin_params())},
        "n_f_evals": int(out["n_f_evals"][0]),
        **{key: out[key].tolist() for key in ("n_steps", "n_accepted", "n_initialized", "status")},
        "ys_sha256": sha(out["ys"]),
        "ys": hexlist(out["ys"]),
    }


def make_tolerance(name, batch, dtype):
    w = to.workloads.make(name, batch=batch, dtype=dtype)
    out = torch_loop.solve(w.f, w.y0, w.t_eval, method=w.method, controller=torch_loop.Controller(**w.controller))
    B, E, F = out["ys"].shape
    g = torch.Generator().manual_seed(0)
    points = torch.stack([torch.randint(0, n, (2048,), generator=g) for n in (B, E, F)], dim=1)
    return {
        "source": f"oracle/torch_loop.py (ATen CPU ops), torch {torch.__version__}, {torch.backends.cpu.get_cpu_capability()}; "
        "tolerance-level vectors (1e-4 mixed absolute / relative)",
        "workload": name,
        "batch": batch,
        "dtype": str(dtype).replace("torch.", ""),
        "method": w.method,
        "controller": w.controller,
        "inputs_sha256": {"y0": sha(w.y0), "t_eval": sha(w.t_eval)},
        "n_f_evals": int(out["n_f_evals"][0]),
        **{key: out[key].tolist() for key in ("n_steps", "n_accepted", "n_initialized", "status")},
        "ys_points": points.tolist(),
        "ys_values": hexlist(out["ys"][points[:, 0], points[:, 1], points[:, 2]]),
        "ys_mean_abs": float(out["ys"].double().abs().mean()).hex(),
    }


if __name__ == "__main__":
    for name, batch, dtype, max_steps in EARLY_STOP_CASES:
        d = make_early_stop(name, batch, dtype, max_steps)
        path = os.path.join(HERE, f"{name}_{d['dtype']}_b{batch}_early_stop.json")
        with open(path, "w") as fh:
            json.dump(d, fh, separators=(",", ":"))
        print(path, os.path.getsize(path), "bytes")
    for name, batch, dtype, method, controller, parts in LOW_ORDER_CASES:
        d = make_low_order(name, batch, dtype, method, controller, parts)
        path = os.path.join(HERE, f"{name}_{d['dtype']}_b{batch}_{method}_{d['controller']['kind']}_low_order.json")
        with open(path, "w") as fh:
            json.dump(d, fh, separators=(",", ":"))
        print(path, os.path.getsize(path), "bytes")
    for name, batch, dtype, method in FIXED_CASES:
        d = make_fixed(name, batch, dtype, method)
        path = os.path.join(HERE, f"{name}_{d['dtype']}_b{batch}_{method}_fixed.json")
        with open(path, "w") as fh:
            json.dump(d, fh, separators=(",", ":"))
        print(path, os.path.getsize(path), "bytes")
    for name, batch, time_dtype, data_dtype in MIXED_CASES:
        d = make_mixed(name, batch, time_dtype, data_dtype)
        path = os.path.join(HERE, f"{name}_t{d['time_dtype'][-2:]}_y{d['data_dtype'][-2:]}_b{batch}_mixed.json")
        with open(path, "w") as fh:
            json.dump(d, fh, separators=(",", ":"))
        print(path, os.path.getsize(path), "bytes")
    for name, batch, dtype in TOLERANCE_CASES:
        d = make_tolerance(name, batch, dtype)
        path = os.path.join(HERE, f"{name}_{d['dtype']}_b{batch}_tolerance.json")
        with open(path, "w") as fh:
            json.dump(d, fh, separators=(",", ":"))
        print(path, os.path.getsize(path), "bytes")
    for name, batch, dtype in CASES:
        d = make(name, batch, dtype)
        path = os.path.join(HERE, f"{name}_{d['dtype']}_b{batch}.json")
        with open(path, "w") as fh:
            json.dump(d, fh, separators=(",", ":"))
        print(path, os.path.getsize(path), "bytes")
