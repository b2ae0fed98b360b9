"""Pins the loop bookkeeping of the ATen-op oracle (oracle/torch_loop.py::run_loop) with the
cases the reference's own suite holds for its loop (tests/adjoint_test.py:26-319), restated
with scripted step / controller callables.  The same cases run against the kernels in
tests/test_protocol_gpu.py.
"""
from itertools import chain, repeat

import numpy as np
import pytest
import torch

from oracle.torch_loop import run_loop

OK, FAILED, MAX_STEPS = 0, 1, 3


def T(x, dtype=torch.float32):
    return torch.as_tensor(x, dtype=dtype)


def curve(t, *idx):
    return (torch.sin(3 * t) + 0.5 * t**2)[..., None]


def script(values):
    values = list(values)
    return chain(values[:-1], repeat(values[-1]))


def scripted(fn, t_eval, dt0, dt, *, accept=(True,), method_status=(None,), controller_status=(None,), t_start=None, t_end=None, y0=None,
             max_steps=None, seen_t=None):  # fmt: skip
    """run_loop with a step that returns fn(t0), a controller that plays back dt / accept, and
    fn itself as the dense output."""
    t_eval = None if t_eval is None else T(t_eval)
    t_start = t_eval[:, 0] if t_start is None else T(t_start)
    t_end = t_eval[:, -1] if t_end is None else T(t_end)
    B = t_start.shape[0]
    y0 = fn(t_start) if y0 is None else y0
    dts, accepts, m_st, c_st = script(dt), script(accept), script(method_status), script(controller_status)
    status = lambda it: (lambda v: None if v is None else T(v, torch.long).expand(B))(next(it))

    def step(running, y, t, dt_, state):
        if seen_t is not None:
            seen_t.append(t)
        return fn(t), fn, state, status(m_st)

    def adapt(t, dt_, y, y1, data, state):
        return T(next(accepts), torch.bool).expand(B), T(next(dts)).expand(B), state, status(c_st)

    keep = lambda mask, new, old: new
    return run_loop(y0, t_start, t_end, t_eval, T(dt0).expand(B), step, adapt, keep, keep, lambda fn_: fn_, None, None, max_steps=max_steps)


def test_evaluation_points_are_hit_exactly():
    t_eval = [[0.0, 2.0], [2.0, 4.0], [0.5, 2.5]]
    ys, status, n_steps, n_acc, n_init, _ = scripted(curve, t_eval, 0.3, [0.3])
    assert status is None and n_steps.tolist() == [7, 7, 7] and n_acc.tolist() == [7, 7, 7] and n_init.tolist() == [2, 2, 2]
    assert torch.equal(ys, curve(T(t_eval)))


def test_samples_step_independently():
    t_eval = [[0.0, 0.15, 1.0], [1.0, 1.9, 2.0]]
    ys, _, n_steps, n_acc, n_init, _ = scripted(curve, t_eval, [0.1, 0.3], [[0.5, 0.125]])
    assert n_steps.tolist() == [3, 7] and n_acc.tolist() == [3, 7] and n_init.tolist() == [3, 3]
    assert torch.equal(ys, curve(T(t_eval)))


def test_several_points_in_one_step_and_on_the_last_step():
    ys, _, n_steps, _, n_init, _ = scripted(curve, [[0.0, 0.25, 0.33, 1.0]], 0.1, [0.5])
    assert n_steps.tolist() == [3] and n_init.tolist() == [4] and torch.equal(ys, curve(T([[0.0, 0.25, 0.33, 1.0]])))
    t_eval = [[0.0, 1.0], [0.9, 1.0], [0.9, 1.0]]
    ys, _, n_steps, n_acc, n_init, _ = scripted(curve, t_eval, [1.1, 1.1, 0.6], [0.6], t_start=[0.0] * 3, t_end=[1.0] * 3)
    assert n_steps.tolist() == [1, 1, 2] and n_acc.tolist() == [1, 1, 2] and n_init.tolist() == [2, 2, 2]
    assert torch.equal(ys, curve(T(t_eval)))


def test_end_point_evaluation_without_evaluation_points():
    # forward Euler on dy/dt = 1 as the step, a line as the dense output
    t_start, t_end, y0 = T([0.0, 5.0, 2.0]), T([10.0, 9.0, 4.5]), T([[0.0], [1.0], [2.0]])
    dt = T([0.5001, 0.2501, 1.0])

    def step(running, y, t, dt_, state):
        y1 = y + dt_[:, None]
        return y1, (t, dt_, y, y1), state, None

    def adapt(t, dt_, y, y1, data, state):
        return torch.ones(3, dtype=torch.bool), dt, state, None

    def line(data):
        t0, h, ya, yb = data
        return lambda tt, idx: ya[idx] + (yb - ya)[idx] * ((tt - t0[idx]) / torch.where(h[idx].abs() > 0, h[idx], 1.0))[:, None]

    keep = lambda mask, new, old: new
    ys, status, n_steps, n_acc, n_init, iterations = run_loop(y0, t_start, t_end, None, dt, step, adapt, keep, keep, line, None, None)
    assert status is None and n_steps.tolist() == [20, 16, 3] and n_acc.tolist() == [20, 16, 3] and n_init.tolist() == [1, 1, 1]
    assert iterations == 20 and ys.shape == (3, 1, 1)
    assert ys[:, 0].numpy() == pytest.approx((y0 + (t_end - t_start)[:, None]).numpy())


def test_max_steps_stops_the_batch():
    y0 = torch.zeros((2, 1))
    const = lambda t, *idx: y0[idx[0]] if idx else y0
    ys, status, n_steps, _, n_init, _ = scripted(const, [[1.0, 4.9], [2.0, 13.0]], 1.0, [1.0], y0=y0, max_steps=7)
    assert status.tolist() == [OK, MAX_STEPS] and n_steps.tolist() == [4, 7] and n_init.tolist() == [2, 1]


def test_rejected_step_is_retried_from_the_same_time():
    seen = []
    accept = [True, [True, False], [True, False], True]
    ys, _, n_steps, n_acc, n_init, _ = scripted(curve, [[0.0, 1.0], [1.0, 2.0]], 0.1, [0.5], accept=accept, seen_t=seen)
    expected = [[0.0, 1.0], [0.1, 1.1], [0.6, 1.1], [1.0, 1.1], [1.0, 1.6]]
    assert torch.stack(seen).numpy() == pytest.approx(np.array(expected))
    assert n_steps.tolist() == [3, 5] and n_acc.tolist() == [3, 3] and n_init.tolist() == [2, 2]
    assert torch.equal(ys, curve(T([[0.0, 1.0], [1.0, 2.0]])))


def test_value_is_stored_only_on_accept():
    calls = iter(range(3))

    def fn(t, *idx):
        if torch.all(t == T(0.6)):
            out = torch.full((3, 1), float(next(calls)))
            return out[idx[0]] if idx else out
        return curve(t)

    accept = [[False, True, True], [False, True, True], [True, True, True]]
    dt = [[1.1, 0.0, 0.5], [1.1, 0.0, 0.0], [0.0] * 3]
    ys, _, n_steps, n_acc, n_init, _ = scripted(fn, [[0.6]] * 3, [1.1, 1.1, 0.55], dt, accept=accept, t_start=[0.0] * 3, t_end=[1.0] * 3)
    assert n_steps.tolist() == [3, 1, 2] and n_acc.tolist() == [1, 1, 2] and n_init.tolist() == [1, 1, 1]
    assert ys.tolist() == [[[2.0]], [[0.0]], [[1.0]]]


def test_rejecting_the_first_step_keeps_the_value_at_t_start():
    y0 = T([[1.3], [2.5]])
    const = lambda t, *idx: y0[idx[0]] if idx else y0
    ys, _, n_steps, n_acc, n_init, _ = scripted(const, [[0.0], [0.0]], 0.6, [0.6], accept=[[False, False], True], t_start=[0.0, 0.0], t_end=[1.0, 2.0], y0=y0)
    assert n_steps.tolist() == [3, 5] and n_acc.tolist() == [2, 4] and n_init.tolist() == [1, 1]
    assert torch.equal(ys, y0[:, None])


def test_failures_stop_every_sample():
    t_eval = [[0.0, 2.0], [2.0, 4.0]]
    _, status, n_steps, n_acc, n_init, _ = scripted(curve, t_eval, 0.2, [0.2], method_status=[[OK, OK]] * 3 + [[OK, FAILED]])
    assert status.tolist() == [OK, FAILED] and n_steps.tolist() == [4, 4] and n_acc.tolist() == [4, 4] and n_init.tolist() == [1, 1]
    _, status, n_steps, _, n_init, _ = scripted(curve, t_eval, 0.2, [0.2], controller_status=[[OK, OK]] * 5 + [[FAILED, OK]])
    assert status.tolist() == [FAILED, OK] and n_steps.tolist() == [6, 6] and n_init.tolist() == [1, 1]
    # both report: the larger code wins
    _, status, _, _, _, _ = scripted(curve, t_eval, 0.2, [0.2], method_status=[[FAILED, OK]], controller_status=[[4, OK]])
    assert status.tolist() == [4, OK]


def test_finished_sample_keeps_its_step_size():
    y0 = torch.zeros((2, 1))
    seen_dt = []

    def step(running, y, t, dt_, state):
        seen_dt.append(dt_)
        return y0, None, state, None

    def adapt(t, dt_, y, y1, data, state):
        return torch.ones(2, dtype=torch.bool), dt_ * T([1.0, 10.0]), state, None  # sample 1 wants to grow

    keep = lambda mask, new, old: new
    run_loop(y0, T([0.0, 0.0]), T([5.0, 0.9]), T([[0.0, 5.0], [0.0, 0.9]]), torch.ones(2), step, adapt, keep, keep,
             lambda d: (lambda tt, idx: y0[idx]), None, None)  # fmt: skip
    assert (torch.stack(seen_dt)[:, 1] < 1.1).all() and len(seen_dt) == 5
