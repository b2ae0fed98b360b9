"""Writes tests/golden/*.json from the scalar C oracle (oracle/erk_oracle.c).

    python tests/golden/make_golden.py

The fixtures are regression vectors of THIS repository's CPU oracle on the seeded
workloads -- inputs are identified by sha256, outputs are the per-sample integer
stats, float64 checksums of ys and the exact ys of a strided subset.  They are not
outputs of the reference implementation (which could not be imported in the
authoring container: its torchtyping dependency is absent there).
"""
import hashlib
import json
import os
import sys

import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

import torchode_amd as to  # noqa: E402
from oracle import c_oracle  # noqa: E402

CASES = [
    ("linear_decay", 256, torch.float64),
    ("linear_decay", 256, torch.float32),
    ("vdp", 512, torch.float32),
    ("vdp", 512, torch.float64),
    ("lorenz", 512, torch.float32),
    ("lorenz", 512, torch.float64),
]


def sha(t: torch.Tensor) -> str:
    return hashlib.sha256(t.contiguous().numpy().tobytes()).hexdigest()


def hexlist(t: torch.Tensor):
    """Exact float values as hex strings (float.hex round-trips through float.fromhex)."""
    return [float(v).hex() for v in t.flatten().tolist()]


def make(name, batch, dtype):
    w = to.workloads.make(name, batch=batch, dtype=dtype)
    cfg = c_oracle.make_config(method=w.method, term=name, nthreads=4, **w.controller)
    out = c_oracle.solve(cfg, w.f.builtin_params(), w.y0, w.t_eval)
    ys = out["ys"].double()
    sub = list(range(0, batch, max(1, batch // 16)))[:16]
    return {
        "workload": name,
        "batch": batch,
        "dtype": str(dtype).replace("torch.", ""),
        "method": w.method,
        "controller": w.controller,
        "inputs_sha256": {"y0": sha(w.y0), "t_eval": sha(w.t_eval), "params": sha(w.f.builtin_params())},
        "n_f_evals": int(out["n_f_evals"][0]),
        "n_steps": out["n_steps"].tolist(),
        "n_accepted": out["n_accepted"].tolist(),
        "n_initialized": out["n_initialized"].tolist(),
        "status": out["status"].tolist(),
        "ys_sum": float(ys.sum()).hex(),
        "ys_sum_sq": float((ys * ys).sum()).hex(),
        "ys_max_abs": float(ys.abs().max()).hex(),
        "subset": sub,
        "ys_subset": hexlist(out["ys"][sub]),
    }


if __name__ == "__main__":
    for name, batch, dtype in CASES:
        d = make(name, batch, dtype)
        path = os.path.join(HERE, f"{name}_{d['dtype']}_b{batch}.json")
        with open(path, "w") as fh:
            json.dump(d, fh, separators=(",", ":"))
        print(path, os.path.getsize(path), "bytes")
