"""tode_solve_builtin_fast_static -- the entry point that allocates nothing, its working memory in a static device
array of the library -- against tode_solve_builtin_fast_sync on the same inputs, through the C ABI.  Bit for bit: ys,
the four int64 stat arrays and the flag block.  Calls come in rows on one stream, a smaller input after a larger one,
so that whatever a call leaves in the array would show in the next."""
import pytest
import torch

import torchode_amd as to

pytestmark = pytest.mark.gpu

F32, F64 = torch.float32, torch.float64


def _args(w, n_eval_given: bool):
    """Argument struct and outputs of one fast solve of workload `w` (tensors on the GPU).  Without evaluation points
    the problem is the workload's time range alone."""
    from torchode_amd import _lib

    B, F = w.y0.shape
    E = w.t_eval.shape[1] if n_eval_given else 0
    params = w.f.builtin_params()
    ys = torch.full((B, max(E, 1), F), float("nan"), dtype=w.y0.dtype, device="cuda")
    out = torch.full((4, B), -7, dtype=torch.int64, device="cuda")
    spec = dict(w.controller)
    kind = spec.pop("kind")
    ctrl = (to.PIDController(**spec) if kind == "pid" else to.IntegralController(**spec)).c_struct()
    a = _lib.SolveArgs()
    a.dtype, a.method, a.term = _lib.DTYPES[w.y0.dtype], {"dopri5": 0, "tsit5": 1}[w.method], w.f.builtin_kind
    a.n_features, a.n_eval, a.n_params, a.batch, a.max_steps, a.iteration_cap = F, E, params.shape[1], B, -1, -1
    scal = list(getattr(w.f, "builtin_scalars", lambda: ())()) + [0.0] * 4
    a.term_scalars = (_lib.C.c_double * 4)(*scal[:4])
    stride = w.t_eval.shape[1]
    a.y0, a.t_start, a.t_end = w.y0.data_ptr(), w.t_eval[:, 0].data_ptr(), w.t_eval[:, -1].data_ptr()
    a.t_eval = w.t_eval.data_ptr() if n_eval_given else None
    a.t_start_stride = a.t_end_stride = stride
    a.params, a.ys = (params.data_ptr() if params.numel() else None), ys.data_ptr()
    keep = [params, ys, out]
    if a.term == _lib.TERM_MLP:
        packed = w.f.builtin_packed(w.y0.device, w.y0.dtype)
        a.shared_params, a.n_shared_params = packed.data_ptr(), packed.numel()
        keep.append(packed)
    return a, ctrl, ys, out, keep


def sync_call(w, n_eval_given=True):
    """The existing entry point: flag words the library allocates, flags on the host when the call returns."""
    from torchode_amd import _lib

    lib = _lib.load()
    a, ctrl, ys, out, keep = _args(w, n_eval_given)
    if not n_eval_given:
        y_idle = torch.full_like(w.y0, float("nan"))
        a.y_idle = y_idle.data_ptr()
        keep.append(y_idle)
    fl = (_lib.C.c_int32 * _lib.FLAG_WORDS)(-1, -1, -1, -1)
    rc = lib.tode_solve_builtin_fast_sync(_lib.C.byref(a), _lib.C.byref(ctrl), *(_lib.ptr(out[i]) for i in range(4)), _lib.stream_of(w.y0), fl)
    _lib.check(rc, "tode_solve_builtin_fast_sync")
    torch.cuda.synchronize()
    return ys, out, list(fl)


def static_call(w, n_eval_given=True, expect=0):
    """The entry point under test: no flag block and no staging area passed in, flags into device memory."""
    from torchode_amd import _lib

    lib = _lib.load()
    a, ctrl, ys, out, keep = _args(w, n_eval_given)
    flags = torch.full((_lib.FLAG_WORDS,), -1, dtype=torch.int32, device="cuda")
    rc = lib.tode_solve_builtin_fast_static(
        _lib.C.byref(a), _lib.C.byref(ctrl), *(_lib.ptr(out[i]) for i in range(4)), flags.data_ptr(), _lib.stream_of(w.y0)
    )
    if expect != 0:
        assert rc == expect, (rc, lib.tode_last_error())
        return lib.tode_last_error().decode()
    _lib.check(rc, "tode_solve_builtin_fast_static")
    torch.cuda.synchronize()
    return ys, out, flags.tolist()


def same(got, want):
    ys_a, out_a, flags_a = got
    ys_b, out_b, flags_b = want
    assert flags_a == flags_b, (flags_a, flags_b)
    assert torch.equal(out_a, out_b)
    assert ys_a.shape == ys_b.shape and bool(((ys_a == ys_b) | (ys_a.isnan() & ys_b.isnan())).all())
    assert not ys_a.isnan().any() and flags_a[3] == 0 and flags_a[0] == int(out_a[0].max())


@pytest.mark.parametrize(
    "name,dtype,sizes",
    [("vdp", F32, (5000, 100, 64)), ("vdp", F64, (3000, 777)), ("lorenz", F32, (300000, 4096, 1)), ("linear_decay", F64, (256, 31))],
)
def test_with_evaluation_points_two_and_more_calls_in_a_row(name, dtype, sizes):
    for batch in sizes:  # the second and later calls are smaller than the one before
        w = to.workloads.make(name, batch=batch, dtype=dtype, device="cuda")
        same(static_call(w), sync_call(w))
    # and the same inputs twice in a row through the static entry point alone
    w = to.workloads.make(name, batch=sizes[0], dtype=dtype, device="cuda")
    first = static_call(w)
    second = static_call(to.workloads.make(name, batch=sizes[-1], dtype=dtype, device="cuda"))
    same(static_call(w), first)
    assert second[2][0] == int(second[1][0].max())


@pytest.mark.parametrize("name,dtype,sizes", [("vdp", F64, (3000, 777)), ("lorenz", F32, (70000, 130)), ("vdp", F32, (4096, 4095))])
def test_without_evaluation_points_the_final_states_are_staged_in_the_static_array(name, dtype, sizes):
    """t_eval=None: the kernel leaves each sample's final state in the staging area and the end point selection,
    enqueued by the same call, picks per sample -- a smaller batch after a larger one finds the larger one's states
    still lying behind its own."""
    for batch in sizes:
        w = to.workloads.make(name, batch=batch, dtype=dtype, device="cuda")
        same(static_call(w, n_eval_given=False), sync_call(w, n_eval_given=False))
    # alternate with and without evaluation points
    w = to.workloads.make(name, batch=sizes[-1], dtype=dtype, device="cuda")
    same(static_call(w), sync_call(w))
    same(static_call(w, n_eval_given=False), sync_call(w, n_eval_given=False))


@pytest.mark.parametrize("name,sizes", [("reaction_diffusion", (24, 5)), ("mlp", (300, 17))])
def test_long_row_kernels_through_the_static_entry_point(name, sizes):
    for batch in sizes:
        w = to.workloads.make(name, batch=batch, dtype=F32, device="cuda")
        same(static_call(w), sync_call(w))


def test_a_batch_that_needs_the_general_kernel_and_the_call_after_it():
    w = to.workloads.make("vdp", batch=200, dtype=F32, device="cuda")
    want = sync_call(w)
    bad = to.workloads.make("vdp", batch=200, dtype=F32, device="cuda")
    bad.t_eval[17, 5] = bad.t_eval[17, 3]  # a row that is not monotone: the kernel asks for the general one
    assert static_call(bad)[2][3] == 1 and sync_call(bad)[2][3] == 1
    same(static_call(w), want)  # the words the flagged call worked on are at their start values again
    empty = w._replace(f=to.VanDerPol(w.f.mu[:0]), y0=w.y0[:0], t_eval=w.t_eval[:0])
    assert static_call(empty)[2] == [0, 2**31 - 1, 0, 0]
    same(static_call(w), want)


def test_sizes_beyond_the_static_array_are_refused_with_a_clear_error():
    from torchode_amd import _lib

    limit = _lib.STATIC_STAGING_BYTES
    most = limit // (3 * 8)  # Lorenz samples in float64 whose final states fit
    big = to.workloads.make("lorenz", batch=most + 1, dtype=F64, device="cuda")
    message = static_call(big, n_eval_given=False, expect=_lib.E_UNSUPPORTED)
    assert "static scratch" in message and str(limit) in message
    assert sync_call(big, n_eval_given=False)[2][3] == 0  # (the entry point with a caller's staging area takes it)
    # with evaluation points the array sets no limit, and the refused call has left nothing behind
    same(static_call(big), sync_call(big))
    at_limit = to.workloads.make("lorenz", batch=most, dtype=F64, device="cuda")
    same(static_call(at_limit, n_eval_given=False), sync_call(at_limit, n_eval_given=False))
    small = to.workloads.make("vdp", batch=500, dtype=F32, device="cuda")
    same(static_call(small, n_eval_given=False), sync_call(small, n_eval_given=False))


def _prepared(w):
    """A static call with every tensor made beforehand: ``launch(stream)`` only enqueues."""
    from torchode_amd import _lib

    lib = _lib.load()
    a, ctrl, ys, out, keep = _args(w, True)
    flags = torch.full((_lib.FLAG_WORDS,), -1, dtype=torch.int32, device="cuda")
    pointers = [_lib.ptr(out[i]) for i in range(4)]

    def launch(stream):
        return lib.tode_solve_builtin_fast_static(_lib.C.byref(a), _lib.C.byref(ctrl), *pointers, flags.data_ptr(), stream)

    return launch, ys, out, flags, keep


def test_calls_leave_the_free_device_memory_as_it_was_and_record_into_a_graph():
    """Nothing is allocated: the free device memory reads the same after a row of calls, and a call records into a HIP
    graph (a capture in the strict mode turns any allocation call into an error); every replay, with eager work and
    synchronisations in between, gives the bits of tode_solve_builtin_fast_sync."""
    from torchode_amd import _lib

    w = to.workloads.make("vdp", batch=5000, dtype=F32, device="cuda")
    want = sync_call(w)
    launch, ys, out, flags, keep = _prepared(w)
    current = _lib.stream_of(w.y0)
    assert launch(current) == 0  # (the first call on the device looks the array's address up)
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    for _ in range(20):
        assert launch(current) == 0
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before
    same((ys, out, flags.tolist()), want)

    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        graph.capture_begin(capture_error_mode="global")
        try:
            rc = launch(_lib.C.c_void_p(side.cuda_stream))
        finally:
            graph.capture_end()
    assert rc == 0, _lib.load().tode_last_error()
    torch.cuda.current_stream().wait_stream(side)
    for replay in range(3):
        ys.fill_(float("nan"))
        out.fill_(-7)
        flags.fill_(-1)
        other = to.workloads.make("lorenz", batch=900 + replay, dtype=F32, device="cuda")  # eager work of another shape in between
        same(static_call(other), sync_call(other))
        graph.replay()
        torch.cuda.synchronize()
        same((ys, out, flags.tolist()), want)
    assert torch.cuda.mem_get_info()[0] <= free_before  # (the test's own tensors aside, nothing was handed back either)


def test_a_call_on_another_stream_is_refused_while_the_last_one_runs():
    from torchode_amd import _lib

    lib = _lib.load()
    w = to.workloads.make("vdp", batch=2000, dtype=F32, device="cuda")
    want = sync_call(w)
    first, *_ = _prepared(w)
    second, ys, out, flags, keep = _prepared(w)
    a, b = torch.cuda.Stream(), torch.cuda.Stream()
    big = torch.randn(8192, 8192, device="cuda")
    torch.cuda.synchronize()
    with torch.cuda.stream(a):
        for _ in range(8):
            big = big @ big * 1e-4  # tens of milliseconds of work in front of the first call
        assert first(_lib.C.c_void_p(a.cuda_stream)) == 0
    rc = second(_lib.C.c_void_p(b.cuda_stream))
    assert rc == _lib.E_UNSUPPORTED and b"another stream" in lib.tode_last_error()
    assert first(_lib.C.c_void_p(a.cuda_stream)) == 0  # the same stream again: ordered by the stream, accepted
    torch.cuda.synchronize()
    assert second(_lib.C.c_void_p(b.cuda_stream)) == 0  # the last call has finished: another stream may have the array
    torch.cuda.synchronize()
    same((ys, out, flags.tolist()), want)
