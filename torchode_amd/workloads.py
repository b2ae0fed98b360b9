"""Seeded synthetic workloads used by the benchmark and the parity tests.

Every random tensor is drawn in float64 on the CPU from one seeded generator,
in a fixed order, then cast to the requested dtype and moved to the requested
device, so that float32 / float64 variants and CPU / GPU runs share the same
underlying values.  ``t_eval`` is ``t0 + (t1 - t0) * (arange(E) / (E - 1))``
computed in float64 and the problem is built from ``t_eval`` alone, so that
``t_start`` / ``t_end`` are exactly its first / last columns.
"""
import math
from typing import NamedTuple, Optional

import torch

from . import builtin_terms as bt


class Workload(NamedTuple):
    name: str
    f: torch.nn.Module  # built-in right-hand side (also a plain torch callable)
    y0: torch.Tensor  # [B, F]
    t_eval: torch.Tensor  # [B, E]
    method: str  # "dopri5" | "tsit5"
    controller: dict  # kind + constructor arguments
    bytes_step: int  # algorithmic HBM bytes per sample-step
    bytes_dense: int  # algorithmic HBM bytes per sample per solve (dense output)


def _uniform(g, a, b, shape):
    return a + (b - a) * torch.rand(shape, generator=g, dtype=torch.float64)


def _log_uniform(g, a, b, shape):
    """exp(U(ln a, ln b)).  The exponential is evaluated with mpmath and rounded once, because
    torch.exp / libm may differ in the last bit between hosts and the workloads have to be
    identical everywhere (parity fixtures identify their inputs by hash)."""
    import mpmath

    u = _uniform(g, math.log(a), math.log(b), shape)
    with mpmath.workprec(100):
        vals = [float(mpmath.exp(mpmath.mpf(v))) for v in u.flatten().tolist()]
    return torch.tensor(vals, dtype=torch.float64).reshape(shape)


def _blur_periodic(u, sigma: float, radius: int):
    """One separable Gaussian blur with periodic boundaries over the last two dims, float64,
    kernel normalised to one (weights through mpmath, for the same reason as above)."""
    import mpmath

    with mpmath.workprec(100):
        w = [float(mpmath.exp(-mpmath.mpf(i * i) / (2 * sigma * sigma))) for i in range(-radius, radius + 1)]
    total = math.fsum(w)
    w = [x / total for x in w]
    for dim in (1, 2):
        acc = torch.zeros_like(u)
        for i, wi in zip(range(-radius, radius + 1), w):
            acc = acc + wi * torch.roll(u, i, dim)
        u = acc
    return u


def _t_eval(t0, t1, E):
    frac = torch.arange(E, dtype=torch.float64) / (E - 1)
    return t0[:, None] + (t1 - t0)[:, None] * frac[None, :]


def _algorithmic_bytes(F, P, C, E, itemsize):
    """One fused pass over a sample's solver state per RK step: y and the FSAL
    derivative in and out, RHS parameters in, controller history in and out,
    (t, dt, t_end) in and (t, dt) out, two int32 counters in and out; the dense
    output writes E*F values and reads E times per solve."""
    step = itemsize * (2 * F + 2 * F + P + 2 * C) + itemsize * 5 + 16
    dense = E * F * itemsize + E * itemsize
    return step, dense


def make(name: str, *, batch: Optional[int] = None, dtype=None, device="cpu") -> Workload:
    """Build workload ``name`` in {"linear_decay", "vdp", "lorenz", "reaction_diffusion", "mlp"}.

    ``batch`` draws the full-size tensors and keeps the first ``batch`` samples
    (samples are independent, so a prefix is a valid smaller instance of the same
    workload)."""
    if name == "linear_decay":
        B, F, E, seed = 256, 4, 10, 101
        dtype = dtype or torch.float64
        g = torch.Generator("cpu").manual_seed(seed)
        k = _log_uniform(g, 0.1, 10.0, (B, F))
        y0 = torch.randn((B, F), generator=g, dtype=torch.float64)
        t_eval = _t_eval(torch.zeros(B, dtype=torch.float64), torch.full((B,), 5.0, dtype=torch.float64), E)
        params, cls = k, bt.LinearDecay
        method, ctrl, P, C = "dopri5", dict(kind="integral", atol=1e-6, rtol=1e-3), F, 0
    elif name == "vdp":
        B, F, E, seed = 65536, 2, 50, 102
        dtype = dtype or torch.float32
        g = torch.Generator("cpu").manual_seed(seed)
        mu = _uniform(g, 0.5, 5.0, (B,))
        y0 = _uniform(g, -2.0, 2.0, (B, F))
        t1 = _uniform(g, 8.0, 12.0, (B,))
        t_eval = _t_eval(torch.zeros(B, dtype=torch.float64), t1, E)
        params, cls = mu, bt.VanDerPol
        method = "tsit5"
        ctrl, P, C = dict(kind="pid", atol=1e-6, rtol=1e-4, pcoeff=0.2, icoeff=0.5, dcoeff=0.0), 1, 2
    elif name == "lorenz":
        B, F, E, seed = 1048576, 3, 20, 103
        dtype = dtype or torch.float32
        g = torch.Generator("cpu").manual_seed(seed)
        rho = _uniform(g, 20.0, 30.0, (B,))
        y0 = torch.randn((B, F), generator=g, dtype=torch.float64) + torch.tensor([0.0, 1.0, 20.0], dtype=torch.float64)
        t_eval = _t_eval(torch.zeros(B, dtype=torch.float64), torch.full((B,), 2.0, dtype=torch.float64), E)
        params, cls = rho, bt.Lorenz63
        method, ctrl, P, C = "dopri5", dict(kind="integral", atol=1e-5, rtol=1e-3), 1, 0
    elif name == "reaction_diffusion":
        B, n, E, seed = 512, 64, 100, 105
        F = n * n
        dtype = dtype or torch.float32
        g = torch.Generator("cpu").manual_seed(seed)
        D = _log_uniform(g, 1e-3, 1e-1, (B,))
        u0 = _blur_periodic(_uniform(g, 0.0, 1.0, (B, n, n)), sigma=2.0, radius=6)
        y0 = u0.reshape(B, F)
        t_eval = _t_eval(torch.zeros(B, dtype=torch.float64), torch.ones(B, dtype=torch.float64), E)
        params, cls = D, bt.ReactionDiffusion
        method = "tsit5"
        ctrl, P, C = dict(kind="pid", atol=1e-5, rtol=1e-3, pcoeff=0.2, icoeff=0.5, dcoeff=0.0), 1, 2
    elif name == "mlp":
        B, F, H, E, seed = 4096, 64, 256, 20, 104
        dtype = dtype or torch.float32
        g = torch.Generator("cpu").manual_seed(seed)
        b1, b2 = math.sqrt(6.0 / (F + 1 + H)), math.sqrt(6.0 / (H + F))
        W1 = _uniform(g, -b1, b1, (H, F + 1))
        W2 = _uniform(g, -b2, b2, (F, H))
        y0 = torch.randn((B, F), generator=g, dtype=torch.float64)
        t_eval = _t_eval(torch.zeros(B, dtype=torch.float64), torch.ones(B, dtype=torch.float64), E)
        method, ctrl, P, C = "dopri5", dict(kind="integral", atol=1e-5, rtol=1e-3), 0, 0
        n = B if batch is None else int(batch)
        assert 0 < n <= B
        w = lambda x: x.to(dtype).contiguous().to(device)
        f = bt.MLPField(w(W1), w(torch.zeros(H, dtype=torch.float64)), w(W2), w(torch.zeros(F, dtype=torch.float64)))
        step, dense = _algorithmic_bytes(F, P, C, E, torch.empty((), dtype=dtype).element_size())
        return Workload(name, f, w(y0[:n]), w(t_eval[:n]), method, ctrl, step, dense)
    else:
        raise ValueError(f"unknown workload {name!r}")

    n = B if batch is None else int(batch)
    assert 0 < n <= B
    cast = lambda x: x[:n].to(dtype).contiguous().to(device)
    f = cls(cast(params))
    step, dense = _algorithmic_bytes(F, P, C, E, torch.empty((), dtype=dtype).element_size())
    return Workload(name, f, cast(y0), cast(t_eval), method, ctrl, step, dense)
