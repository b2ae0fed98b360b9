"""Pins for the two CPU oracles (oracle/torch_loop.py: the loop as ATen operations;
oracle/erk_oracle.c: the scalar C restatement).

Nothing here retypes an oracle formula.  Each function is checked against what
the mathematics or an independent library fixes: order conditions and stability
polynomials of the tableaux, scipy's RK45 coefficients and start-step routine,
numpy.polynomial for the dense output, the linear test equation for a whole RK
step, hand-computed controller cases from the reference's own tests, the exact
integer stats the reference's README prints, and finally the two oracles against
each other (they share no code: one is batched ATen ops, the other scalar C).
"""
import ctypes
import math
from fractions import Fraction

import numpy as np
import pytest
import torch
from numpy.polynomial import Polynomial

import torchode_amd as to
from helpers import aten_host_matches
from oracle import c_oracle, torch_loop as tl

F32, F64 = torch.float32, torch.float64

needs_pinned_aten = pytest.mark.skipif(
    not aten_host_matches(), reason="this host's ATen CPU kernels round differently from the host the oracle was pinned on"
)


# --------------------------------------------------------------------------- #
# tableaux                                                                    #
# --------------------------------------------------------------------------- #


def c_tableau(method):
    class Tab(ctypes.Structure):
        _fields_ = [("c", ctypes.c_double * 7), ("a", (ctypes.c_double * 7) * 7), ("b", ctypes.c_double * 7),
                    ("b_err", ctypes.c_double * 7), ("b_other", (ctypes.c_double * 7) * 3), ("n_other", ctypes.c_int)]  # fmt: skip

    fn = c_oracle.lib().oracle_get_tableau
    fn.restype = ctypes.POINTER(Tab)
    t = fn(c_oracle.METHODS[method]).contents
    n = t.n_other
    return dict(c=np.array(t.c), a=np.array([list(r) for r in t.a]), b=np.array(t.b), b_err=np.array(t.b_err),
                b_other=np.array([list(r) for r in t.b_other])[:n])  # fmt: skip


def torch_tableau(method):
    t = tl.TABLEAUX[method]
    return dict(c=t.c.numpy(), a=t.a.numpy(), b=t.b.numpy(), b_err=t.b_err.numpy(), b_other=t.b_other.numpy())


def poly_coeffs(a, w):
    """coefficients of sum_m z^m w^T A^(m-1) 1, m = 1..7"""
    v, out = np.ones(7), []
    for _ in range(7):
        out.append(float(w @ v))
        v = a @ v
    return out


STABILITY = {
    "dopri5": [1, 1 / 2, 1 / 6, 1 / 24, 1 / 120, 1 / 600, 0],
    "tsit5": [1, 1 / 2, 1 / 6, 1 / 24, 1 / 120, 0.0014322113248073473, 0],
}
ERROR_POLY = {
    "dopri5": [0, 0, 0, 0, -5.388888888888905e-4, 2.166666666666667e-4, -2.7777777777777776e-5],
    "tsit5": [0, 0, 0, 0, -4.264763677523328e-4, 1.5595331976679983e-4, -2.1700171587990116e-5],
}


@pytest.mark.parametrize("source", [c_tableau, torch_tableau], ids=["c", "torch"])
@pytest.mark.parametrize("method", ["dopri5", "tsit5"])
def test_tableau_invariants(method, source):
    t = source(method)
    c, a, b, be = t["c"], t["a"], t["b"], t["b_err"]
    assert np.allclose(a.sum(1), c, atol=1e-15)
    assert np.all(np.triu(a) == 0)  # explicit
    assert np.array_equal(a[6], b) and c[6] == 1.0 and c[0] == 0.0  # FSAL + SSAL
    assert abs(b.sum() - 1) < 1e-15 and abs(be.sum()) < 1e-16
    for q in range(1, 5):  # quadrature order conditions of a 5th order method
        assert abs(b @ c**q - 1 / (q + 1)) < 1e-15
    assert abs(b @ (a @ c) - 1 / 6) < 1e-15 and abs(b @ (a @ (a @ c)) - 1 / 24) < 1e-15
    # stability polynomial and error polynomial on y' = lambda y
    assert np.allclose(poly_coeffs(a, b), STABILITY[method], atol=2e-16, rtol=1e-13)
    assert np.allclose(poly_coeffs(a, be), ERROR_POLY[method], atol=2e-15, rtol=1e-11)


@pytest.mark.parametrize("source", [c_tableau, torch_tableau], ids=["c", "torch"])
def test_dopri5_is_scipys_rk45(source):
    from scipy.integrate._ivp.rk import RK45

    t = source("dopri5")
    assert np.allclose(t["c"][:6], RK45.C, atol=1e-16)
    assert np.allclose(t["a"][:6, :5], RK45.A, atol=1e-15)
    assert np.allclose(t["b"][:6], RK45.B, atol=1e-16)
    # the reference's embedded weights give 2/3 of the classical Dormand-Prince error estimate
    # (its 7th low-order weight is 1/60 where the textbook pair has 1/40); scipy's E is b_low - b
    assert np.allclose(t["b_err"], -2.0 / 3.0 * RK45.E, atol=1e-16)
    # mid-point weights: sum = 1/2 and first moment 1/8 (a 4th order value at t + dt/2)
    mid = t["b_other"][0]
    assert abs(mid.sum() - 0.5) < 1e-15 and abs(mid @ t["c"] - 0.125) < 1e-15


@pytest.mark.parametrize("source", [c_tableau, torch_tableau], ids=["c", "torch"])
def test_tsit5_dense_weights_by_brute_force(source):
    """Multiply out the seven factored basis polynomials with numpy.polynomial."""
    t = source("tsit5")
    P = Polynomial
    x = P([0, 1])
    basis = [
        -1.0530884977290216 * x * (x - 1.3299890189751412) * (x**2 - 1.4364028541716351 * x + 0.7139816917074209),
        0.1017 * x**2 * (x**2 - 2.1966568338249754 * x + 1.2949852507374631),
        2.490627285651252793 * x**2 * (x**2 - 2.38535645472061657 * x + 1.57803468208092486),
        -16.54810288924490272 * (x - 1.21712927295533244) * (x - 0.61620406037800089) * x**2,
        47.37952196281928122 * (x - 1.203071208372362603) * (x - 0.658047292653547382) * x**2,
        -34.87065786149660974 * (x - 1.2) * (x - 0.666666666666666667) * x**2,
        2.5 * (x - 1) * (x - 0.6) * x**2,
    ]
    w = t["b_other"]
    for s, p in enumerate(basis):
        coef = np.zeros(5)
        coef[: len(p.coef)] = p.coef
        assert abs(coef[0]) < 1e-15
        assert abs(coef[1] - (1.0 if s == 0 else 0.0)) < 1e-15  # theta^1 row is (1, 0, ..., 0)
        assert np.allclose(w[:, s], coef[2:], rtol=1e-14, atol=1e-15)
    # the interpolant at theta = 1 is the 5th order solution: sum_p W[p][s] + [s == 0] == b[s]
    assert np.allclose(w.sum(0) + np.eye(7)[0], t["b"], atol=2e-14)


# What tsit5.py:11-50 evaluates to under sympy 1.14: the factored basis polynomials with floating point
# literals, expanded and collected in t, each coefficient through float().  Two entries of the t^3 row (stages
# 4 and 6) are one unit in the last place away from the exact expansion rounded once.
TSIT5_DENSE_WEIGHTS = [
    [-2.763706197274826, 0.13169999999999998, 3.930296236894751, -12.411077166933676, 37.50931341651104,
     -27.896526289197286, 1.5],
    [2.9132554618219126, -0.2234, -5.941033872131505, 30.338188630282318, -88.1789048947664, 65.09189467479368, -4.0],
    [-1.0530884977290216, 0.1017, 2.490627285651253, -16.548102889244902, 47.37952196281928, -34.87065786149661, 2.5],
]  # fmt: skip


def kernel_tsit5_weights():
    """The constants compiled into the HIP library (a host-side table read, no GPU needed)."""
    from torchode_amd import _lib

    lib = _lib.load()
    c, a, be = (ctypes.c_double * 7)(), (ctypes.c_double * 49)(), (ctypes.c_double * 7)()
    other, n = (ctypes.c_double * 21)(), ctypes.c_int32(0)
    tsit5 = 1  # TODE_TSIT5
    assert lib.tode_tableau(tsit5, c, a, be, other, ctypes.byref(n)) == 0 and n.value == 3
    return np.array(list(other)).reshape(3, 7)


def test_tsit5_dense_weights_are_the_float_derivation_literally():
    """All 21 weights, in the ATen-op oracle (which runs the sympy float derivation), the C oracle and the
    kernels: equal as floats, not approximately."""
    derived, first = tl.tsit5_dense_weights()
    assert derived == TSIT5_DENSE_WEIGHTS
    assert first == [0.9999999999999999, 0.0, 0.0, 0.0, 0.0, 0.0, 0.0]
    assert c_tableau("tsit5")["b_other"].tolist() == TSIT5_DENSE_WEIGHTS
    assert torch_tableau("tsit5")["b_other"].tolist() == TSIT5_DENSE_WEIGHTS
    assert kernel_tsit5_weights().tolist() == TSIT5_DENSE_WEIGHTS


def test_tsit5_float_derivation_differs_from_the_exact_expansion_in_two_last_places():
    """Guards the derivation itself: expanding in exact rationals and rounding once gives other last digits
    in exactly two places, so a derivation that silently went exact (or reordered) would show here."""
    import sympy as sp

    th = sp.Symbol("t")
    R = lambda x: sp.Rational(Fraction(float(x)))
    basis = [
        R(-1.0530884977290216) * th * (th - R(1.3299890189751412)) * (th**2 - R(1.4364028541716351) * th + R(0.7139816917074209)),
        R(0.1017) * th**2 * (th**2 - R(2.1966568338249754) * th + R(1.2949852507374631)),
        R(2.490627285651252793) * th**2 * (th**2 - R(2.38535645472061657) * th + R(1.57803468208092486)),
        R(-16.54810288924490272) * (th - R(1.21712927295533244)) * (th - R(0.61620406037800089)) * th**2,
        R(47.37952196281928122) * (th - R(1.203071208372362603)) * (th - R(0.658047292653547382)) * th**2,
        R(-34.87065786149660974) * (th - R(1.2)) * (th - R(0.666666666666666667)) * th**2,
        R(2.5) * (th - 1) * (th - R(0.6)) * th**2,
    ]  # fmt: skip
    exact = [[float(sp.Poly(sp.expand(b), th).coeff_monomial(th**p)) for b in basis] for p in (2, 3, 4)]
    differing = [(p, s) for p in range(3) for s in range(7) if exact[p][s] != TSIT5_DENSE_WEIGHTS[p][s]]
    assert differing == [(1, 3), (1, 5)]
    for p, s in differing:
        assert abs(exact[p][s] - TSIT5_DENSE_WEIGHTS[p][s]) <= 2 * np.spacing(abs(exact[p][s]))


# --------------------------------------------------------------------------- #
# one RK step: the linear test equation                                       #
# --------------------------------------------------------------------------- #


@pytest.mark.parametrize("method", ["dopri5", "tsit5"])
def test_rk_step_on_linear_test_equation(method):
    """y' = -k y: one step gives y1 = R(z) y0 and err = E(z) y0 with z = -k dt."""
    rng = np.random.default_rng(5)
    k = torch.tensor(rng.uniform(0.1, 3.0, 4))
    y0 = torch.tensor(rng.normal(size=4))
    dt, t0 = 0.37, 1.25
    z = (-k * dt).numpy()
    R = 1 + sum(c * z ** (m + 1) for m, c in enumerate(STABILITY[method]))
    E = sum(c * z ** (m + 1) for m, c in enumerate(ERROR_POLY[method]))
    # C oracle
    cfg = c_oracle.make_config(method=method, term="linear_decay", kind="integral", atol=1e-6, rtol=1e-3)
    k0 = c_oracle.rhs(cfg, k, t0, y0)
    assert torch.allclose(k0, -k * y0, rtol=0, atol=0)
    y1, err, ks = c_oracle.erk_step(cfg, k, t0, dt, y0, k0)
    assert np.allclose(y1.numpy(), R * y0.numpy(), rtol=1e-14)
    assert np.allclose(err.numpy(), E * y0.numpy(), rtol=1e-7, atol=1e-16)
    assert torch.equal(ks[0], k0) and torch.allclose(ks[6], -k * y1, rtol=1e-15)
    # ATen-op oracle
    tab = tl.TABLEAUX[method].cast(F64, F64)
    f = lambda t, y: (-k) * y
    y1t, errt, kt = tl.erk_step(f, tab, torch.tensor([t0], dtype=F64), torch.tensor([dt], dtype=F64), y0[None], k0[None])
    assert np.allclose(y1t[0].numpy(), R * y0.numpy(), rtol=1e-14)
    assert np.allclose(errt[0].numpy(), E * y0.numpy(), rtol=1e-7, atol=1e-16)
    # (a one-sample batch takes ATen's small-matrix kernels, so the two oracles agree here to
    # rounding only; bit-for-bit agreement is tested on realistic batch sizes further down)
    assert torch.allclose(y1t[0], y1, rtol=1e-14) and torch.allclose(kt[:, 0], ks, rtol=1e-12)


def test_rk_step_evaluates_at_the_nodes():
    """reference tests/single_step_methods_test.py:22-53, on the Dopri5 nodes."""
    seen = []

    def f(t, y):
        seen.append(t.clone())
        return y

    tab = tl.TABLEAUX["dopri5"].cast(F64, F64)
    t0, dt = torch.tensor([0.5, -1.0], dtype=F64), torch.tensor([0.25, 0.5], dtype=F64)
    tl.erk_step(f, tab, t0, dt, torch.ones(2, 1, dtype=F64), torch.ones(2, 1, dtype=F64))
    assert len(seen) == 6  # FSAL: the first stage is reused
    for i, t in enumerate(seen, start=1):
        assert torch.allclose(t, t0 + tab.c[i] * dt)


# --------------------------------------------------------------------------- #
# controllers: hand-computed cases from the reference's tests                 #
# --------------------------------------------------------------------------- #


def both_adapt(kind_kwargs, dt, y0, y1, err, prev=1.0, prev_prev=1.0, order=5):
    """Run adapt in both oracles on one sample; returns (c_result, torch_result)."""
    cfg = c_oracle.make_config(method="dopri5", term="vdp", **kind_kwargs)
    c = c_oracle.adapt(cfg, dt, y0, y1, err, prev, prev_prev)
    ctrl = tl.Controller(**kind_kwargs)
    dtype = y0.dtype
    a, dn, st, r, p, pp = tl.adapt(ctrl, order, torch.tensor([dt], dtype=dtype), y0[None], y1[None], err[None],
                                   torch.tensor([prev], dtype=dtype), torch.tensor([prev_prev], dtype=dtype))  # fmt: skip
    t = dict(ratio=r.item(), accept=bool(a.item()), dt_next=dn.item(), status=int(st.item()), prev=p.item(), prev_prev=pp.item())
    return c, t


@pytest.mark.parametrize("kind", [dict(kind="integral", atol=1.0, rtol=0.0), dict(kind="pid", atol=1.0, rtol=0.0, pcoeff=0.0, icoeff=1.0, dcoeff=0.0)])
def test_error_ratio_and_factor_hand_case(kind):
    """atol=1, rtol=0, err=(0.5, 0.5): rms ratio 0.5, factor 0.9 * 0.5**(-1/5), accepted."""
    y = torch.tensor([1.0, 2.0], dtype=F64)
    err = torch.tensor([0.5, -0.5], dtype=F64)
    for res in both_adapt(kind, 1.0, y, y, err):
        assert res["ratio"] == pytest.approx(0.5, rel=1e-15)
        assert res["accept"] and res["status"] == 0
        assert res["dt_next"] == pytest.approx(0.9 * 0.5 ** (-0.2), rel=1e-14)


def test_rtol_uses_larger_of_y0_y1_and_float32_tolerances():
    y0 = torch.tensor([1.0, -4.0], dtype=F64)
    y1 = torch.tensor([-3.0, 2.0], dtype=F64)
    err = torch.tensor([3e-4, 4e-4], dtype=F64)
    kind = dict(kind="integral", atol=1e-6, rtol=1e-4)
    a32, r32 = float(np.float32(1e-6)), float(np.float32(1e-4))  # the reference keeps them in float32 buffers
    q = np.array([3e-4 / (a32 + r32 * 3.0), 4e-4 / (a32 + r32 * 4.0)])
    expect = math.sqrt((q**2).mean())
    exact_tol = math.sqrt((np.array([3e-4 / (1e-6 + 1e-4 * 3.0), 4e-4 / (1e-6 + 1e-4 * 4.0)]) ** 2).mean())
    for res in both_adapt(kind, 0.1, y0, y1, err):
        assert res["ratio"] == pytest.approx(expect, rel=1e-14)
        assert abs(res["ratio"] - exact_tol) > 1e-9 * expect  # float32 rounding of the tolerances is visible


def test_zero_error_gives_finite_step_and_max_factor():
    """reference tests/step_size_controllers_test.py:50-62"""
    y = torch.tensor([1.0, 2.0, 3.0], dtype=F32)
    for kind in (dict(kind="integral", atol=1.0, rtol=0.0), dict(kind="pid", atol=1.0, rtol=1.0, pcoeff=1.0, icoeff=1.0, dcoeff=1.0)):
        for res in both_adapt(kind, 1.0, y, y, torch.zeros(3)):
            assert math.isfinite(res["dt_next"]) and res["dt_next"] == pytest.approx(10.0)
            assert res["ratio"] == pytest.approx(1e-38, rel=1e-6) and res["accept"]


def test_infinite_and_nan_norm_signal_status_4():
    """reference tests/step_size_controllers_test.py:73-122"""
    kind = dict(kind="pid", atol=1.0, rtol=1.0, pcoeff=1.0, icoeff=1.0, dcoeff=1.0)
    y = torch.ones(2)
    big = torch.tensor([torch.finfo(F32).max, 1.0])
    for res in both_adapt(kind, 1.0, y, y, big):
        assert res["status"] == 4 and not res["accept"]
    ynan = torch.tensor([float("nan"), 1.0])
    for res in both_adapt(kind, 1.0, ynan, ynan, torch.ones(2)):
        assert res["status"] == 4 and not res["accept"]
    for res in both_adapt(kind, 1.0, y, y, torch.tensor([0.5, 1.25])):
        assert res["status"] == 0


def test_pid_history_shifts_on_accept_and_freezes_on_reject():
    """reference tests/step_size_controllers_test.py:132-163, 209-242"""
    kind = dict(kind="pid", atol=0.75, rtol=0.0, pcoeff=0.0, icoeff=1.0, dcoeff=0.0, safety=1.0)
    y = torch.tensor([1.0, 2.0, 3.0])
    for res in both_adapt(kind, 1.0, y, y, torch.tensor([0.0, 1.6, 0.0]), prev=0.3, prev_prev=0.7):
        assert not res["accept"] and res["dt_next"] < 1.0
        assert res["prev"] == pytest.approx(0.3) and res["prev_prev"] == pytest.approx(0.7)
    for res in both_adapt(kind, 1.0, y, y, torch.zeros(3) + 0.1, prev=0.3, prev_prev=0.7):
        assert res["accept"] and res["dt_next"] > 1.0
        assert res["prev"] == pytest.approx(res["ratio"]) and res["prev_prev"] == pytest.approx(0.3)


def test_pid_factor_closed_form():
    kind = dict(kind="pid", atol=1.0, rtol=0.0, pcoeff=0.2, icoeff=0.5, dcoeff=0.1, factor_max=1e9, factor_min=0.0)
    y = torch.tensor([1.0, 1.0], dtype=F64)
    err = torch.tensor([0.3, 0.3], dtype=F64)
    kI, kP, kD = 0.5 / 5, 0.2 / 5, 0.1 / 5
    expect = 0.9 * 0.3 ** (-(kI + kP + kD)) * 0.6 ** (kP + 2 * kD) * 0.8 ** (-kD)
    for res in both_adapt(kind, 2.0, y, y, err, prev=0.6, prev_prev=0.8):
        assert res["dt_next"] == pytest.approx(2.0 * expect, rel=1e-13)


def test_dt_min_and_dt_max():
    """reference tests/step_size_controllers_test.py:181-206, 252-271"""
    y = torch.tensor([3.0, 4.0])
    kind = dict(kind="integral", atol=1.0, rtol=0.0, factor_min=0.0, dt_min=0.5)
    for res in both_adapt(kind, 1.0, y, y, torch.tensor([0.0, 100.0]), order=2):
        pass
    cfg_res, t_res = both_adapt(kind, 1.0, y, y, torch.tensor([0.0, 100.0]))
    for res in (cfg_res, t_res):
        assert not res["accept"] and res["status"] == 2 and res["dt_next"] == pytest.approx(0.5)
    kind = dict(kind="integral", atol=1.0, rtol=0.0, dt_max=0.4)
    for res in both_adapt(kind, 1.0, y, y, torch.tensor([0.5, 0.5])):
        assert res["accept"] and res["dt_next"] == pytest.approx(0.4) and res["status"] == 0
    for res in both_adapt(kind, -1.0, y, y, torch.tensor([0.5, 0.5])):  # sign is kept
        assert res["dt_next"] == pytest.approx(-0.4)


# --------------------------------------------------------------------------- #
# pow                                                                         #
# --------------------------------------------------------------------------- #


@pytest.mark.parametrize("dtype", [F32, F64], ids=["f32", "f64"])
def test_pow_reproduces_torch_pow_bit_for_bit(dtype):
    """The oracle restates the SLEEF pow that ATen's vectorised CPU kernels call; on the vector
    body of a tensor (length a multiple of 16) the results must be identical to torch.pow."""
    g = torch.Generator().manual_seed(7)
    n = 1 << 18
    for p in (-0.2, -0.14, 0.04, 0.2, -0.12, 0.08, -0.02, 0.5000001):  # the controllers' range of exponents
        x = torch.exp(torch.empty(n, dtype=torch.float64).uniform_(-87.0, 10.0, generator=g)).to(dtype)
        x[:4] = torch.tensor([1e-38, 1.0, 0.5, 3.0], dtype=dtype)  # subnormal in float32, exact 1, ...
        assert torch.equal(c_oracle.pow_array(x, p), x**p), p
    for p in (1.7, -2.3):  # larger exponents, bases such that the result stays a normal number
        x = torch.exp(torch.empty(n, dtype=torch.float64).uniform_(-20.0, 20.0, generator=g)).to(dtype)
        assert torch.equal(c_oracle.pow_array(x, p), x**p), p
    near_one = (1 + torch.empty(n, dtype=torch.float64).uniform_(-1e-3, 1e-3, generator=g)).to(dtype)
    assert torch.equal(c_oracle.pow_array(near_one, -0.14), near_one**-0.14)


def test_pow_accuracy_and_special_cases():
    import mpmath as mp

    mp.mp.prec = 200
    rng = np.random.default_rng(11)
    worst = 0.0
    for _ in range(2000):
        x = float(10 ** rng.uniform(-38, 3))
        p = float(rng.choice([-0.2, -0.14, 0.04, 0.2, -0.1, 0.08, 1.7, -2.3]))
        got = c_oracle.pow_scalar(x, p)
        ref = mp.power(mp.mpf(x), mp.mpf(p))
        worst = max(worst, float(abs((mp.mpf(got) - ref) / ref)))
    assert worst < 2.3e-16  # within one ulp of the exact value in float64
    for dtype in (F32, F64):
        P = lambda x, y: c_oracle.pow_scalar(x, y, dtype)
        assert P(1.0, 0.3) == 1.0 and P(7.0, 0.0) == 1.0 and P(float("nan"), 0.0) == 1.0
        assert P(0.0, 0.5) == 0.0 and P(0.0, -0.5) == math.inf
        assert P(math.inf, -0.2) == 0.0 and P(math.inf, 0.2) == math.inf and math.isnan(P(float("nan"), 0.2))
        assert P(4.0, 0.5) == pytest.approx(2.0, rel=1e-6) and P(1e-38, -0.2) == pytest.approx(1e7 * 10**0.6, rel=1e-5)
        for x, y in ((0.0, 0.2), (math.inf, -0.14), (2.0, math.inf), (0.5, math.inf), (1.0, math.inf)):
            t = torch.tensor([x], dtype=dtype) ** y
            assert P(x, y) == t.item(), (x, y)


# --------------------------------------------------------------------------- #
# start step: scipy's select_initial_step                                     #
# --------------------------------------------------------------------------- #


@pytest.mark.parametrize("kind", ["integral", "pid"])
def test_initial_step_reduces_to_scipy(kind):
    from scipy.integrate._ivp.common import select_initial_step

    rng = np.random.default_rng(3)
    spec = dict(kind=kind, atol=1e-6, rtol=1e-4)
    if kind == "pid":
        spec.update(pcoeff=0.2, icoeff=0.5, dcoeff=0.0)
    a32, r32 = float(np.float32(1e-6)), float(np.float32(1e-4))
    cfg = c_oracle.make_config(method="tsit5", term="vdp", **spec)
    for _ in range(25):
        mu = float(rng.uniform(0.5, 5))
        y0 = rng.uniform(-2, 2, 2)
        t0 = float(rng.uniform(-1, 1))
        direction = float(rng.choice([-1.0, 1.0]))
        t1 = t0 + direction * float(rng.uniform(1, 10))
        fun = lambda t, y: np.array([y[1], mu * (1 - y[0] * y[0]) * y[1] - y[0]])
        # scipy's error-estimator order 4 <=> exponent 1/5 <=> torchode's convergence order 5
        try:
            h = select_initial_step(fun, t0, y0, t1, np.inf, fun(t0, y0), direction, 4, r32, a32)
        except TypeError:  # older signature without t_bound
            h = select_initial_step(fun, t0, y0, fun(t0, y0), direction, 4, r32, a32)
        dt_c, f0 = c_oracle.initial_step(cfg, torch.tensor([mu], dtype=F64), t0, torch.tensor(y0), t1)
        assert dt_c == pytest.approx(direction * h, rel=1e-12)
        assert np.allclose(f0.numpy(), fun(t0, y0), rtol=1e-15)
        f = to.VanDerPol(torch.tensor([mu], dtype=F64))
        dt_t, _ = tl.initial_step(f, tl.Controller(**spec), 5, torch.tensor([t0], dtype=F64), torch.tensor(y0)[None],
                                  torch.tensor([int(direction)]), torch.tensor([abs(t1 - t0)], dtype=F64))  # fmt: skip
        assert dt_t.item() == pytest.approx(direction * h, rel=1e-12)


def test_initial_step_zero_interval_differs_between_controllers():
    """The integral copy maps h0 == 0 to d2 = inf (step 0); the PID copy divides 0/0 (NaN)."""
    y0 = torch.tensor([0.3, -1.1], dtype=F64)
    mu = torch.tensor([1.5], dtype=F64)
    ci = c_oracle.make_config(method="tsit5", term="vdp", kind="integral", atol=1e-6, rtol=1e-4)
    cp = c_oracle.make_config(method="tsit5", term="vdp", kind="pid", atol=1e-6, rtol=1e-4, pcoeff=0.2, icoeff=0.5)
    assert c_oracle.initial_step(ci, mu, 2.0, y0, 2.0)[0] == 0.0
    assert math.isnan(c_oracle.initial_step(cp, mu, 2.0, y0, 2.0)[0])
    f = to.VanDerPol(mu)
    args = (5, torch.tensor([2.0], dtype=F64), y0[None], torch.tensor([-1]), torch.tensor([0.0], dtype=F64))
    assert tl.initial_step(f, tl.Controller("integral", 1e-6, 1e-4), *args)[0].item() == 0.0
    assert math.isnan(tl.initial_step(f, tl.Controller("pid", 1e-6, 1e-4, 0.2, 0.5, 0.0), *args)[0].item())


# --------------------------------------------------------------------------- #
# dense output                                                                #
# --------------------------------------------------------------------------- #


def _one_real_step(method, dtype=F64):
    w = to.workloads.make("vdp", batch=1, dtype=dtype)
    cfg = c_oracle.make_config(method=method, term="vdp", kind="integral", atol=1e-6, rtol=1e-4)
    mu, y0 = w.f.mu, w.y0[0]
    k0 = c_oracle.rhs(cfg, mu, 0.0, y0)
    dt = 0.2
    y1, err, k = c_oracle.erk_step(cfg, mu, 0.0, dt, y0, k0)
    return cfg, mu, y0, y1, k, dt


@needs_pinned_aten
@pytest.mark.parametrize("method", ["dopri5", "tsit5"])
def test_quartic_hermite_identities(method):
    cfg, mu, y0, y1, k, dt = _one_real_step(method)
    q = c_oracle.quartic(cfg, dt, y0, y1, k).numpy()  # lowest power first
    p = [Polynomial(q[:, f]) for f in range(2)]
    for f in range(2):
        assert p[f](0.0) == y0[f].item()
        assert p[f].deriv()(0.0) == pytest.approx(dt * k[0, f].item(), rel=1e-15)
        assert p[f](1.0) == pytest.approx(y1[f].item(), rel=1e-12)
        assert p[f].deriv()(1.0) == pytest.approx(dt * k[6, f].item(), rel=1e-9, abs=1e-12)
    if method == "dopri5":
        mid = tl.TABLEAUX["dopri5"].b_other[0].numpy()
        for f in range(2):
            assert p[f](0.5) == pytest.approx(y0[f].item() + dt * float(mid @ k[:, f].numpy()), rel=1e-13)
    # evaluation: Horner on (t - t0) / dt, checked with numpy
    t0 = 1.5
    for t in (1.5, 1.55, 1.7):
        out = c_oracle.quartic_eval(torch.tensor(q), t0, dt, t).numpy()
        x = (t - t0) / ((t0 + dt) - t0)
        assert np.allclose(out, [p[0](x), p[1](x)], rtol=1e-14)
    # the ATen-op oracle builds the same coefficients, bit for bit
    tab = tl.TABLEAUX[method].cast(F64, F64)
    dtt = torch.tensor([dt], dtype=F64)
    coeff = tl.quartic_tsit5(tab, dtt, y0[None], k[:, None]) if method == "tsit5" else tl.quartic_dopri5(tab, dtt, y0[None], y1[None], k[:, None])
    assert np.array_equal(np.stack([c[0].numpy() for c in coeff]), q)


def test_quartic_with_zero_dt_has_no_nan():
    """reference tests/interpolation_test.py:46-51"""
    q = torch.rand(5, 2, dtype=F64)
    out = c_oracle.quartic_eval(q, 1.0, 0.0, 1.0)
    assert not torch.isnan(out).any() and torch.equal(out, q[0])
    coeff = tuple(q[i][None] for i in range(5))
    out_t = tl.quartic_eval(coeff, torch.tensor([1.0]), torch.tensor([1.0]), torch.tensor([1.0]), torch.tensor([0]))
    assert torch.equal(out_t[0], q[0])


def test_tsit5_recovers_a_quartic():
    """reference tests/interpolation_test.py:105-127: stages sampled from the derivative of a
    known quartic give back its coefficients (abs 5e-4 in float32)."""
    t0, dt = 1.0, 1.5
    p = Polynomial([1, -0.5, 1.2, 3.3, 0.5], domain=(t0, t0 + dt), window=(0, 1))
    c = tl.TABLEAUX["tsit5"].c.numpy()
    k = torch.tensor(np.stack([p.deriv()(t0 + ci * dt) for ci in c]))[:, None].float()
    y0 = torch.tensor([p(t0)]).float()
    y1 = torch.tensor([p(t0 + dt)]).float()
    cfg = c_oracle.make_config(method="tsit5", term="vdp", kind="integral", atol=1e-6, rtol=1e-4)
    q = c_oracle.quartic(cfg, dt, y0, y1, k)
    assert q[:, 0].numpy() == pytest.approx(p.coef, abs=5e-4)


# --------------------------------------------------------------------------- #
# whole loop                                                                  #
# --------------------------------------------------------------------------- #


def test_readme_example_stats():
    """README.md:57-59 prints the exact stats of this solve."""
    y0 = torch.tensor([[1.2], [5.0]])
    t_eval = torch.stack((torch.linspace(0, 5, 10), torch.linspace(3, 4, 10)))
    out = tl.solve(lambda t, y: -0.5 * y, y0, t_eval, method="dopri5", controller=tl.Controller("integral", 1e-6, 1e-3))
    assert out["n_f_evals"].tolist() == [26, 26]
    assert out["n_steps"].tolist() == [4, 2] and out["n_accepted"].tolist() == [4, 2]
    assert out["n_initialized"].tolist() == [10, 10] and out["status"].tolist() == [0, 0]
    # same problem through the C oracle (linear decay with k = 0.5)
    cfg = c_oracle.make_config(method="dopri5", term="linear_decay", kind="integral", atol=1e-6, rtol=1e-3)
    c = c_oracle.solve(cfg, torch.full((2, 1), 0.5), y0, t_eval)
    assert c["n_steps"].tolist() == [4, 2] and c["n_f_evals"].tolist() == [26, 26] and c["n_initialized"].tolist() == [10, 10]
    assert torch.allclose(c["ys"], out["ys"], rtol=2e-4)
    assert torch.allclose(out["ys"][0, :, 0], 1.2 * torch.exp(-0.5 * t_eval[0]), rtol=2e-3)


@pytest.mark.parametrize("ctrl", [tl.Controller("pid", 1e-5, 1e-5, 0.0, 1.0, 0.0), tl.Controller("integral", 1e-5, 1e-5)])
def test_constant_dynamics_both_directions(ctrl):
    """reference tests/adjoint_test.py:357-368: exact values, one sample forwards, one backwards."""
    y0 = torch.tensor([[1.0], [9.0]])
    t_eval = torch.tensor([[0.0, 3.0, 5.0], [2.0, 0.5, -8.0]])
    out = tl.solve(lambda t, y: 2 * torch.ones_like(y), y0, t_eval, method="dopri5", controller=ctrl)
    assert out["ys"].squeeze(-1).numpy() == pytest.approx(np.array([[1.0, 7.0, 11.0], [9.0, 6.0, -11.0]]))
    assert (out["n_f_evals"] == 2 + 6 * out["n_steps"].max()).all()


def test_linear_decay_closed_form_and_invariants():
    w = to.workloads.make("linear_decay")
    cfg = c_oracle.make_config(method=w.method, term="linear_decay", nthreads=4, **w.controller)
    out = c_oracle.solve(cfg, w.f.builtin_params(), w.y0, w.t_eval)
    exact = w.y0[:, None, :] * torch.exp(-w.f.k[:, None, :] * w.t_eval[:, :, None])
    assert ((out["ys"] - exact).abs() <= 1e-2 * exact.abs() + 1e-4).all()  # tolerance-level accuracy (rtol 1e-3)
    assert (out["n_accepted"] <= out["n_steps"]).all() and (out["status"] == 0).all()
    assert (out["n_f_evals"] == 2 + 6 * out["n_steps"].max()).all()
    assert torch.equal(out["ys"][:, 0], w.y0)  # first point is t_start: exact copy


def test_batch_composition_independence():
    """docs/comparison.md:12-17: a sample's result does not depend on who else is in the batch."""
    w = to.workloads.make("vdp", batch=96, dtype=F64)
    cfg = c_oracle.make_config(method=w.method, term="vdp", nthreads=4, **w.controller)
    full = c_oracle.solve(cfg, w.f.builtin_params(), w.y0, w.t_eval)
    idx = torch.tensor([3, 17, 40, 95])
    sub = c_oracle.solve(cfg, w.f.builtin_params()[idx], w.y0[idx], w.t_eval[idx])
    assert torch.equal(sub["ys"], full["ys"][idx]) and torch.equal(sub["n_steps"], full["n_steps"][idx])
    assert sub["n_f_evals"][0] <= full["n_f_evals"][0]  # only the batch-uniform evaluation counter differs


@needs_pinned_aten
def test_max_steps_global_stop_semantics():
    """reference tests/adjoint_test.py:121-135: the sample that exhausts max_steps gets status 3,
    everybody stops at that iteration, finished samples keep status 0."""
    w = to.workloads.make("vdp", batch=64, dtype=F64)
    ctrl = tl.Controller(**w.controller)
    free = tl.solve(w.f, w.y0, w.t_eval, method=w.method, controller=ctrl)
    cap = int(free["n_steps"].median())
    out = tl.solve(w.f, w.y0, w.t_eval, method=w.method, controller=ctrl, max_steps=cap)
    assert out["n_steps"].max().item() == cap
    done = free["n_steps"] < cap
    assert (out["status"][done] == 0).all() and (out["status"][~done] == 3).all()
    assert (out["n_initialized"][~done] < 50).any()
    cfg = c_oracle.make_config(method=w.method, term="vdp", max_steps=cap, **w.controller)
    c = c_oracle.solve(cfg, w.f.builtin_params(), w.y0, w.t_eval)
    for key in ("n_steps", "n_accepted", "n_initialized", "status", "n_f_evals"):
        assert torch.equal(c[key], out[key]), key


# --------------------------------------------------------------------------- #
# the two oracles against each other                                          #
# --------------------------------------------------------------------------- #


@needs_pinned_aten
@pytest.mark.parametrize("dtype", [F32, F64], ids=["f32", "f64"])
@pytest.mark.parametrize("name,batch", [("linear_decay", 128), ("vdp", 192), ("lorenz", 192)])
def test_c_oracle_equals_aten_oracle_bit_for_bit(name, batch, dtype):
    """The scalar C loop and the batched ATen-op loop agree to the last bit on every output.
    This pins every arithmetic choice of the C oracle (fused or not, order of sums, true
    division, reciprocal-then-multiply, the pow routine) against ATen's CPU kernels.
    Batch sizes are multiples of 16 with B*F >= 200: ATen's own arithmetic is different on the
    scalar tail of a tensor (libm pow) and for tiny matrices (unfused stage sums)."""
    w = to.workloads.make(name, batch=batch, dtype=dtype)
    a = tl.solve(w.f, w.y0, w.t_eval, method=w.method, controller=tl.Controller(**w.controller))
    cfg = c_oracle.make_config(method=w.method, term=name, nthreads=4, **w.controller)
    c = c_oracle.solve(cfg, w.f.builtin_params(), w.y0, w.t_eval)
    for key in ("n_steps", "n_accepted", "n_initialized", "status", "n_f_evals"):
        assert torch.equal(a[key], c[key]), key
    assert torch.equal(a["ys"], c["ys"])


@needs_pinned_aten
@pytest.mark.parametrize("method,kind", [("dopri5", dict(kind="pid", atol=1e-6, rtol=1e-4, pcoeff=0.3, icoeff=0.4, dcoeff=0.1)),
                                         ("tsit5", dict(kind="integral", atol=1e-7, rtol=1e-5))])  # fmt: skip
def test_oracles_agree_for_other_method_controller_pairs(method, kind):
    # (B*F must be >= 200: below that ATen's matrix product for the stage sums takes a
    # different small-matrix kernel and no longer evaluates the fused chain)
    w = to.workloads.make("vdp", batch=160, dtype=F64)
    a = tl.solve(w.f, w.y0, w.t_eval, method=method, controller=tl.Controller(**kind))
    c = c_oracle.solve(c_oracle.make_config(method=method, term="vdp", **kind), w.f.builtin_params(), w.y0, w.t_eval)
    assert torch.equal(a["ys"], c["ys"]) and torch.equal(a["n_steps"], c["n_steps"]) and torch.equal(a["n_accepted"], c["n_accepted"])


@needs_pinned_aten
def test_oracles_agree_without_t_eval_and_backwards():
    w = to.workloads.make("linear_decay", batch=96, dtype=F64)
    ts, te = w.t_eval[:, -1].contiguous() * 0.2, w.t_eval[:, 0].contiguous()
    a = tl.solve(w.f, w.y0, None, t_start=ts, t_end=te, method=w.method, controller=tl.Controller(**w.controller))
    cfg = c_oracle.make_config(method=w.method, term="linear_decay", **w.controller)
    c = c_oracle.solve(cfg, w.f.builtin_params(), w.y0, None, t_start=ts, t_end=te)
    assert torch.equal(a["ys"], c["ys"]) and torch.equal(a["n_steps"], c["n_steps"]) and (c["n_initialized"] == 1).all()


@needs_pinned_aten
@pytest.mark.parametrize("dtype", [F32, F64], ids=["f32", "f64"])
def test_oracles_agree_on_a_larger_van_der_pol_batch(dtype):
    w = to.workloads.make("vdp", batch=2048, dtype=dtype)
    a = tl.solve(w.f, w.y0, w.t_eval, method=w.method, controller=tl.Controller(**w.controller))
    c = c_oracle.solve(c_oracle.make_config(method=w.method, term="vdp", nthreads=4, **w.controller), w.f.builtin_params(), w.y0, w.t_eval)
    assert torch.equal(a["ys"], c["ys"])
    for key in ("n_steps", "n_accepted", "n_initialized", "status", "n_f_evals"):
        assert torch.equal(a[key], c[key]), key


@needs_pinned_aten
def test_aten_results_depend_on_batch_size_the_oracle_does_not():
    """Documented property of the substrate, not of the solver: ATen's elementwise kernels
    process 32 values per iteration with fused vector code and the remaining tail with scalar
    code that rounds differently, and tiny batches go through a different matrix kernel, so
    ATen's per-sample results change with the batch a sample is in.  The C oracle (and the
    kernels) always use the vector-body / large-matrix arithmetic."""
    w = to.workloads.make("vdp", batch=2048, dtype=F32)
    ctrl = tl.Controller(**w.controller)
    full = tl.solve(w.f, w.y0, w.t_eval, method=w.method, controller=ctrl)
    n = 2048 - 5  # 2043 = 63 * 32 + 27: the last 27 samples are on the scalar tail
    part = tl.solve(to.VanDerPol(w.f.mu[:n]), w.y0[:n], w.t_eval[:n], method=w.method, controller=ctrl)
    assert torch.equal(part["ys"][:2016], full["ys"][:2016])  # vector body: independent of the batch
    assert not torch.equal(part["ys"][2016:], full["ys"][2016:n])  # tail: ATen disagrees with itself
    cfg = c_oracle.make_config(method=w.method, term="vdp", **w.controller)
    c_part = c_oracle.solve(cfg, w.f.builtin_params()[:n], w.y0[:n], w.t_eval[:n])
    assert torch.equal(c_part["ys"], full["ys"][:n])  # the oracle reproduces the full-batch values for every sample


@needs_pinned_aten
def test_headline_configuration_at_full_size():
    """Van der Pol, B=65536, float32, Tsit5 + PID: the scalar C oracle reproduces the loop issued
    as ATen CPU operations bit for bit -- every ys value and every integer stat of all 65536
    samples (bars: 1e-4 and 99.9 %)."""
    w = to.workloads.make("vdp")
    a = tl.solve(w.f, w.y0, w.t_eval, method=w.method, controller=tl.Controller(**w.controller))
    c = c_oracle.solve(c_oracle.make_config(method=w.method, term="vdp", nthreads=8, **w.controller), w.f.builtin_params(), w.y0, w.t_eval)
    assert torch.equal(a["ys"], c["ys"])
    for key in ("n_steps", "n_accepted", "n_initialized", "status", "n_f_evals"):
        assert torch.equal(a[key], c[key]), key


@needs_pinned_aten
@pytest.mark.parametrize("seed", [1000, 1001, 1002, 1004, 1008, 1010, 1014, 1017, 1019, 1021])
def test_oracles_agree_on_random_configurations(seed):
    """The seeded random configurations of the GPU suites (term, shapes, per-sample time spans with evaluation
    points outside them, tolerances, controller coefficients; linear systems partly backwards in time): scalar C loop
    against the batched ATen-op loop, on a whole number of 32-sample vector bodies."""
    from test_persistent_gpu import _random_case

    f, y0, t_eval, t_start, t_end, method, controller = _random_case(seed)
    n = y0.shape[0] // 32 * 32
    assert n * y0.shape[1] >= 200, "pick seeds with batches large enough for ATen's fused matrix kernels"
    f = type(f)(f.builtin_params()[:n].reshape(n, -1) if type(f) is to.LinearDecay else f.builtin_params()[:n, 0])
    y0, t_eval, t_start, t_end = y0[:n], t_eval[:n], t_start[:n], t_end[:n]
    a = tl.solve(f, y0, t_eval, method=method, controller=tl.Controller(**controller), t_start=t_start, t_end=t_end, max_steps=4000)
    from helpers import c_oracle_solve

    c = c_oracle_solve(f, y0, t_eval, method, controller, t_start=t_start, t_end=t_end, max_steps=4000, nthreads=4)
    for key in ("n_steps", "n_accepted", "n_initialized", "status", "n_f_evals"):
        assert torch.equal(a[key], c[key]), key
    # (a point beyond t_end is never written, and where a later point of its row is, the reference's searchsorted
    # counts it as initialised all the same: compare what was written)
    written = c["written"]
    assert torch.equal(a["ys"][written], c["ys"][written]) and not c["ys"][written].isnan().any()
    assert (~written).float().mean() < 0.1 and c["ys"][~written].isnan().all()


@needs_pinned_aten
@pytest.mark.parametrize("seed", range(12))
def test_oracles_agree_where_the_controller_powers_are_shortcuts(seed):
    """PID coefficients that make the controller's exponents -1, 2, 3, -2 or -0.5, which ATen computes by reciprocal,
    products and reciprocal square root instead of pow (tests/helpers.py::shortcut_case)."""
    from helpers import c_oracle_solve, shortcut_case

    f, y0, t_eval, t_start, t_end, method, ctrl, max_steps, dt0 = shortcut_case(seed)
    a = tl.solve(f, y0, t_eval, method=method, controller=tl.Controller(**ctrl), t_start=t_start, t_end=t_end, dt0=dt0, max_steps=max_steps)
    c = c_oracle_solve(f, y0, t_eval, method, ctrl, t_start=t_start, t_end=t_end, dt0=dt0, max_steps=max_steps, nthreads=4)
    for key in ("n_steps", "n_accepted", "n_initialized", "status", "n_f_evals"):
        assert torch.equal(a[key], c[key]), key
    av, cv = a["ys"][c["written"]], c["ys"][c["written"]]
    assert bool(((av == cv) | (av.isnan() & cv.isnan())).all())
    assert int(c["n_steps"].max()) > 20


@needs_pinned_aten
@pytest.mark.parametrize("seed", range(24))
def test_oracles_agree_on_wild_configurations(seed):
    """Scalar C loop against the batched ATen-op loop over everything the loop knows at once: evaluation points
    shuffled within rows or absent, dt_min / dt_max, a small max_steps, a user's first step (tests/helpers.py::wild_case)."""
    from helpers import c_oracle_solve, wild_case

    f, y0, t_eval, t_start, t_end, method, ctrl, max_steps, dt0 = wild_case(seed)
    a = tl.solve(f, y0, t_eval, method=method, controller=tl.Controller(**ctrl), t_start=t_start, t_end=t_end, dt0=dt0, max_steps=max_steps)
    c = c_oracle_solve(f, y0, t_eval, method, ctrl, t_start=t_start, t_end=t_end, dt0=dt0, max_steps=max_steps, nthreads=4)
    for key in ("n_steps", "n_accepted", "n_initialized", "status", "n_f_evals"):
        assert torch.equal(a[key], c[key]), key
    av, cv = a["ys"][c["written"]], c["ys"][c["written"]]
    assert bool(((av == cv) | (av.isnan() & cv.isnan())).all())


@needs_pinned_aten
@pytest.mark.parametrize("seed", range(24, 40))
def test_oracles_agree_on_wild_configurations_with_non_finite_samples(seed):
    """The same with three samples NaN, infinite, huge or blowing up later (tests/helpers.py::poisoned)."""
    from helpers import c_oracle_solve, poisoned, wild_case

    f, y0, t_eval, t_start, t_end, method, ctrl, max_steps, dt0 = wild_case(seed)
    y0 = poisoned(y0, seed)
    max_steps = min(max_steps, 400)
    a = tl.solve(f, y0, t_eval, method=method, controller=tl.Controller(**ctrl), t_start=t_start, t_end=t_end, dt0=dt0, max_steps=max_steps)
    c = c_oracle_solve(f, y0, t_eval, method, ctrl, t_start=t_start, t_end=t_end, dt0=dt0, max_steps=max_steps, nthreads=4)
    for key in ("n_steps", "n_accepted", "n_initialized", "status", "n_f_evals"):
        assert torch.equal(a[key], c[key]), key
    av, cv = a["ys"][c["written"]], c["ys"][c["written"]]
    assert bool(((av == cv) | (av.isnan() & cv.isnan())).all())
    assert seed % 4 == 3 or (c["status"] != 0).any()  # (a sample that is merely large may solve after all)


# --------------------------------------------------------------------------- #
# the low-order methods of the ATen-op oracle                                 #
# --------------------------------------------------------------------------- #


def test_heun_step_and_hermite_cubic():
    """Heun on y' = lambda y: y1 = (1 + z + z^2/2) y0 and err = (z^2/2) y0 with z = lambda dt (the second-order
    stability polynomial against the first-order one); the cubic dense output takes y0, y1 and both end slopes."""
    lam = torch.tensor([[-0.7, 0.3], [2.0, -5.0]], dtype=F64)
    y0, t0, dt = torch.tensor([[1.5, -2.0], [0.25, 3.0]], dtype=F64), torch.tensor([0.2, -1.0], dtype=F64), torch.tensor([0.4, -0.05], dtype=F64)
    y1, err, k = tl.erk_step_general(lambda t, y: lam * y, tl._heun(), t0, dt, y0)
    z = lam * dt[:, None]
    assert torch.allclose(y1, (1 + z + z * z / 2) * y0, rtol=1e-14, atol=0) and torch.allclose(err, (z * z / 2) * y0, rtol=1e-13, atol=1e-18)
    coeff, idx, eps = tl.cubic_from_k(dt, y0, y1, k), torch.arange(2), 1e-6
    at = lambda x: tl.cubic_eval(coeff, t0, t0 + dt, t0 + x * dt, idx)
    assert torch.equal(at(0.0), y0) and torch.allclose(at(1.0), y1, rtol=1e-15, atol=0)
    assert torch.allclose((at(eps) - at(0.0)) / eps, dt[:, None] * k[0], rtol=1e-4) and torch.allclose((at(1.0) - at(1.0 - eps)) / eps, dt[:, None] * k[1], rtol=1e-4)
    line = lambda x: tl.linear_eval(t0, dt, y0, y1, t0 + x * dt, idx)
    assert torch.equal(line(0.0), y0) and torch.allclose(line(1.0), y1, rtol=1e-15, atol=0) and torch.allclose(line(0.5), (y0 + y1) / 2, rtol=1e-15, atol=0)


def test_low_order_solves_against_the_analytic_solution_and_the_reference_step_counts():
    """reference tests/fixed_step_controller_test.py:9-19 (analytic solution to 1e-2), tests/adjoint_test.py:98-118
    (Euler, no evaluation points: n_steps [20, 16, 3]); evaluation counts 2 per Heun step, 1 per Euler step."""
    w = to.workloads.make("linear_decay", batch=64, dtype=F64)
    exact = w.y0[:, None] * torch.exp(-w.f.k[:, None] * (w.t_eval - w.t_eval[:, :1])[:, :, None])
    heun = tl.solve_low_order(w.f, w.y0, w.t_eval, method="heun", controller=tl.Controller("pid", 1e-6, 1e-4, 0.2, 0.5, 0.0))
    assert (heun["ys"] - exact).abs().max() < 1e-4 and int(heun["n_f_evals"][0]) == 2 + 2 * int(heun["n_steps"].max()) and (heun["n_steps"] > 20).all()
    dt0 = torch.full((64,), 1e-3, dtype=F64)
    for method, per_step in (("heun", 2), ("euler", 1)):
        out = tl.solve_low_order(w.f, w.y0, w.t_eval, method=method, controller=tl.Controller("fixed", 0.0, 0.0), dt0=dt0)
        assert (out["ys"] - exact).abs().max() < 1e-2 and int(out["n_f_evals"][0]) == per_step * int(out["n_steps"].max())
    no_estimate = tl.solve_low_order(w.f, w.y0, w.t_eval, method="euler", controller=tl.Controller("integral", 1e-6, 1e-4), dt0=dt0 * 10)
    assert torch.equal(no_estimate["n_steps"], no_estimate["n_accepted"]) and (no_estimate["status"] == 0).all()  # accepted as is, step kept
    y0 = torch.tensor([[0.0], [1.0], [2.0]], dtype=F64)
    t_start, t_end = torch.tensor([0.0, 5.0, 2.0], dtype=F64), torch.tensor([10.0, 9.0, 4.5], dtype=F64)
    steps = torch.tensor([0.5001, 0.2501, 1.0], dtype=F64)
    out = tl.solve_low_order(lambda t, y: torch.ones_like(y), y0, None, method="euler", controller=tl.Controller("fixed", 0.0, 0.0), t_start=t_start, t_end=t_end, dt0=steps)
    assert out["n_steps"].tolist() == [20, 16, 3] and torch.allclose(out["ys"][:, 0], y0 + (t_end - t_start)[:, None], rtol=1e-12)


@pytest.mark.parametrize("dtype", [F32, F64], ids=["f32", "f64"])
def test_tensor_to_a_python_float_follows_atens_shortcuts(dtype):
    """``x ** p`` with a Python float ``p`` is not always pow: ATen fills for 0, copies for 1, takes the reciprocal
    square root, the reciprocal and plain products for -0.5, -1, 2, 3, -2 (step_size_controllers.py:292-293 and 612-617
    reach these with order-2 methods or unusual PID coefficients).  The oracle's version reproduces each of them bit for
    bit, special values included; 0.5 is ATen's square root kernel, which on some hosts comes from a vector math library
    and is then off by one ulp for under 2 % of arguments."""
    g = torch.Generator().manual_seed(5)
    n = 1 << 15  # (whole vectors: the scalar tail of ATen's kernels is another implementation)
    x = torch.rand(n, dtype=dtype, generator=g) * 10 + 1e-3
    x[:8] = torch.tensor([0.0, 1.0, float("inf"), float("nan"), 1e-30, 1e30, 2.0, 0.25], dtype=dtype)
    for p in (0.0, 1.0, -1.0, 2.0, 3.0, -2.0, -0.5):
        got, want = c_oracle.pow_tensor_scalar(x, p), x**p
        assert torch.equal(got.isnan(), want.isnan()) and torch.equal(got.nan_to_num(nan=0.0), want.nan_to_num(nan=0.0)), p
        if p not in (0.0, 1.0):
            generic = c_oracle.pow_array(x, p)
            assert not torch.equal(generic.nan_to_num(nan=0.0), want.nan_to_num(nan=0.0)), p  # the shortcut is not a no-op
    got, want = c_oracle.pow_tensor_scalar(x, 0.5), x**0.5
    assert torch.equal(got.nan_to_num(nan=-1.0), torch.from_numpy(np.sqrt(x.numpy())).nan_to_num(nan=-1.0))
    off = (got != want) & ~want.isnan()
    assert off.double().mean() < 0.02 and torch.allclose(got[8:], want[8:], rtol=4 * torch.finfo(dtype).eps, atol=0)
