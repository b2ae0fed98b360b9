"""TEST INFRASTRUCTURE ONLY -- ctypes access to the scalar C oracle (erk_oracle.c).

Loads ``oracle/liberk_oracle.so`` (built by ``make -C oracle`` or by
``__graft_entry__.build()``) and exposes the whole-solve entry point plus the
single-function entry points used by the pin tests.  Inputs and outputs are
CPU torch tensors.
"""
import ctypes as C
import os
import subprocess
from typing import Optional

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "liberk_oracle.so")

METHODS = {"dopri5": 0, "tsit5": 1}
CONTROLLERS = {"integral": 0, "pid": 1}
TERMS = {"linear_decay": 0, "vdp": 1, "lorenz": 2}


class Config(C.Structure):
    _fields_ = [
        ("method", C.c_int32),
        ("controller", C.c_int32),
        ("term", C.c_int32),
        ("nthreads", C.c_int32),
        ("atol", C.c_double),
        ("rtol", C.c_double),
        ("pcoeff", C.c_double),
        ("icoeff", C.c_double),
        ("dcoeff", C.c_double),
        ("safety", C.c_double),
        ("factor_min", C.c_double),
        ("factor_max", C.c_double),
        ("has_dt_min", C.c_int32),
        ("has_dt_max", C.c_int32),
        ("dt_min", C.c_double),
        ("dt_max", C.c_double),
        ("max_steps", C.c_int64),
    ]


def build(force: bool = False) -> str:
    if force or not os.path.exists(_SO):
        subprocess.run(["make", "-C", _HERE, "-B", "liberk_oracle.so"], check=True, capture_output=True)
    return _SO


_lib = None


def lib():
    global _lib
    if _lib is None:
        _lib = C.CDLL(build())
        _lib.oracle_pow.restype = C.c_double
        _lib.oracle_pow.argtypes = [C.c_double, C.c_double]
        _lib.oracle_powf.restype = C.c_float
        _lib.oracle_powf.argtypes = [C.c_float, C.c_float]
        _lib.oracle_initial_step_f32.restype = C.c_float
        _lib.oracle_initial_step_f64.restype = C.c_double
    return _lib


def make_config(
    *,
    method: str,
    term: str,
    kind: str,
    atol: float,
    rtol: float,
    pcoeff: float = 0.0,
    icoeff: float = 1.0,
    dcoeff: float = 0.0,
    dt_min: Optional[float] = None,
    dt_max: Optional[float] = None,
    safety: float = 0.9,
    factor_min: float = 0.2,
    factor_max: float = 10.0,
    max_steps: Optional[int] = None,
    nthreads: int = 1,
) -> Config:
    return Config(
        METHODS[method],
        CONTROLLERS[kind],
        TERMS[term],
        nthreads,
        atol,
        rtol,
        pcoeff,
        icoeff,
        dcoeff,
        safety,
        factor_min,
        factor_max,
        dt_min is not None,
        dt_max is not None,
        dt_min or 0.0,
        dt_max or 0.0,
        -1 if max_steps is None else max_steps,
    )


def _sfx(dtype):
    return {torch.float32: "f32", torch.float64: "f64"}[dtype]


def _p(t):
    return None if t is None else C.c_void_p(t.data_ptr())


def _real(dtype):
    return C.c_float if dtype == torch.float32 else C.c_double


def pow_scalar(x: float, p: float, dtype=torch.float64) -> float:
    """pow(x, p) of the oracle in `dtype` (one value)."""
    return lib().oracle_powf(x, p) if dtype == torch.float32 else lib().oracle_pow(x, p)


def pow_array(x: torch.Tensor, p: float) -> torch.Tensor:
    """Elementwise x ** p of the oracle (p is rounded to x's dtype, as ATen does)."""
    x = x.contiguous()
    out = torch.empty_like(x)
    if x.dtype == torch.float32:
        lib().oracle_powf_array(_p(x), C.c_float(p), _p(out), C.c_int64(x.numel()))
    else:
        lib().oracle_pow_array(_p(x), C.c_double(p), _p(out), C.c_int64(x.numel()))
    return out


def pow_tensor_scalar(x: torch.Tensor, p: float) -> torch.Tensor:
    """``x ** p`` for a Python float ``p`` with ATen's special exponents (0, 1, 0.5, -0.5, -1, 2, 3, -2) computed the
    way its CPU kernels compute them."""
    x = x.contiguous()
    out = torch.empty_like(x)
    fn = lib().oracle_rpowf_array if x.dtype == torch.float32 else lib().oracle_rpow_array
    fn(_p(x), C.c_double(p), _p(out), C.c_int64(x.numel()))
    return out


def solve(cfg: Config, params, y0, t_eval=None, *, t_start=None, t_end=None, dt0=None, trace_iters=0, trace_B=0):
    """Whole solve on the CPU.  ``ys`` rows that the loop never wrote are NaN."""
    dtype = y0.dtype
    B, F = y0.shape
    if t_start is None:
        t_start = t_eval[:, 0]
    if t_end is None:
        t_end = t_eval[:, -1]
    E = 0 if t_eval is None else t_eval.shape[1]
    y0, params = y0.contiguous(), params.reshape(B, -1).to(dtype).contiguous()
    t_start, t_end = t_start.contiguous(), t_end.contiguous()
    t_eval = None if t_eval is None else t_eval.contiguous()
    dt0 = None if dt0 is None else dt0.contiguous()
    ys = torch.full((B, max(E, 1), F), float("nan"), dtype=dtype)
    i64 = lambda: torch.zeros(B, dtype=torch.int64)
    n_steps, n_acc, n_init, status = i64(), i64(), i64(), i64()
    n_f = C.c_int64(0)
    written = torch.ones((B, max(E, 1)), dtype=torch.uint8)  # (without evaluation points: the end point, always)
    trace = torch.zeros((trace_iters, trace_B, 4), dtype=dtype) if trace_iters else None
    fn = getattr(lib(), f"oracle_solve_{_sfx(dtype)}")
    rc = fn(
        C.byref(cfg), C.c_int64(B), C.c_int(F), C.c_int(E), _p(y0), _p(t_start), _p(t_end), _p(t_eval), _p(dt0),
        _p(params), C.c_int(params.shape[1]), _p(ys), _p(n_steps), _p(n_acc), _p(n_init), _p(status), C.byref(n_f),
        _p(trace), C.c_int64(trace_iters), C.c_int64(trace_B), _p(written),
    )  # fmt: skip
    assert rc == 0
    out = dict(
        ts=t_eval if t_eval is not None else t_end[:, None],
        ys=ys,
        status=status,
        n_f_evals=torch.full((B,), n_f.value, dtype=torch.int64),
        n_steps=n_steps,
        n_accepted=n_acc,
        n_initialized=n_init,
        written=written.bool(),  # which rows of ys the loop stored (n_initialized is the reference's searchsorted over these marks)
    )
    if trace is not None:
        out["trace"] = trace
    return out


# ---- single-function entry points (one sample at a time) ----------------------------


def rhs(cfg, par, t, y):
    dy = torch.empty_like(y)
    getattr(lib(), f"oracle_rhs_{_sfx(y.dtype)}")(C.byref(cfg), _p(par), _real(y.dtype)(t), _p(y), _p(dy), C.c_int(y.numel()))
    return dy


def erk_step(cfg, par, t0, dt, y0, k0):
    F = y0.numel()
    k = torch.empty(7, F, dtype=y0.dtype)
    y1, err = torch.empty_like(y0), torch.empty_like(y0)
    R = _real(y0.dtype)
    getattr(lib(), f"oracle_erk_step_{_sfx(y0.dtype)}")(
        C.byref(cfg), _p(par), R(t0), R(dt), _p(y0), _p(k0), _p(k), _p(y1), _p(err), C.c_int(F)
    )
    return y1, err, k


def adapt(cfg, dt, y0, y1, err, prev=1.0, prev_prev=1.0):
    out = torch.empty(6, dtype=y0.dtype)
    R = _real(y0.dtype)
    getattr(lib(), f"oracle_adapt_{_sfx(y0.dtype)}")(
        C.byref(cfg), R(dt), _p(y0), _p(y1), _p(err), R(prev), R(prev_prev), _p(out), C.c_int(y0.numel())
    )
    return dict(ratio=out[0].item(), accept=bool(out[1].item()), dt_next=out[2].item(), status=int(out[3].item()),
                prev=out[4].item(), prev_prev=out[5].item())  # fmt: skip


def initial_step(cfg, par, t0, y0, t_end):
    f0 = torch.empty_like(y0)
    R = _real(y0.dtype)
    dt = getattr(lib(), f"oracle_initial_step_{_sfx(y0.dtype)}")(C.byref(cfg), _p(par), R(t0), _p(y0), R(t_end), _p(f0), C.c_int(y0.numel()))
    return dt, f0


def quartic(cfg, dt, y0, y1, k):
    F = y0.numel()
    q = torch.empty(5, F, dtype=y0.dtype)
    getattr(lib(), f"oracle_quartic_{_sfx(y0.dtype)}")(C.byref(cfg), _real(y0.dtype)(dt), _p(y0), _p(y1), _p(k.contiguous()), _p(q), C.c_int(F))
    return q


def quartic_eval(q, t0, dt, t):
    F = q.shape[1]
    out = torch.empty(F, dtype=q.dtype)
    R = _real(q.dtype)
    getattr(lib(), f"oracle_quartic_eval_{_sfx(q.dtype)}")(_p(q.contiguous()), R(t0), R(dt), R(t), _p(out), C.c_int(F))
    return out
