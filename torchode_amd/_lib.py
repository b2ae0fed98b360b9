"""ctypes binding of libtorchode_amd.so (declared in include/torchode_amd.h).

The library is loaded from this directory; if it is absent it is built once with
hipcc.  There is no fallback: when the library cannot be loaded, or the tensors
are not on a HIP device, the callers raise.
"""
import ctypes as C
import os
import threading

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libtorchode_amd.so")

ABI_VERSION = 23
END_ONLY_MAX_BATCH = 2048 * 64  # TODE_END_ONLY_MAX_BATCH
MLP_PACKED_SIZE = {"float32": 152 * 256, "bfloat16": 92 * 256}
MLP_INPUTS = {"float32": 0, "bfloat16": 1}
F32, F64 = 0, 1
DOPRI5, TSIT5, HEUN, EULER = 0, 1, 2, 3
CTRL_INTEGRAL, CTRL_PID, CTRL_FIXED = 0, 1, 2
TERM_REACTION_DIFFUSION, TERM_MLP = 3, 4
PERSISTENT_TERMS = (0, 1, 2, 3, 4)  # TODE_TERM_* that a whole-solve kernel evaluates itself
GENERAL_TERMS = (0, 1, 2)  # ... of which these also have the general kernel (every case, not only the common one)
FLAG_MAX_ITERATIONS, FLAG_FIRST_FAILURE, FLAG_NON_MONOTONE, FLAG_NEEDS_GENERAL, FLAG_WORDS = 0, 1, 2, 3, 4
INT32_MAX = 2**31 - 1

DTYPES = {torch.float32: F32, torch.float64: F64}
E_INVALID, E_UNSUPPORTED, E_HIP = -1, -2, -3  # return codes (TODE_E_*)
STATIC_STAGING_BYTES = 2 << 20  # TODE_STATIC_STAGING_BYTES

# every symbol include/torchode_amd.h declares
EXPORTS = (
    "tode_abi_version",
    "tode_source_hash",
    "tode_last_error",
    "tode_solve_builtin",
    "tode_solve_builtin_fast",
    "tode_solve_builtin_fast_sync",
    "tode_solve_builtin_fast_static",
    "tode_solve_builtin_auto",
    "tode_solve_builtin_backward",
    "tode_solve_backward_scratch_bytes",
    "tode_solve_workspace_bytes",
    "tode_mlp_pack_weights",
    "tode_mlp_pack_weights_for",
    "tode_select_end_point",
    "tode_step_begin",
    "tode_step_stage",
    "tode_step_finish",
    "tode_step_finish_backward",
    "tode_step_stage_backward",
    "tode_step_stats",
    "tode_finalize_stats",
    "tode_set_fast_kernel_variant",
    "tode_set_kernel_timing",
    "tode_last_solve_kernel_ms",
    "tode_last_solve_kernel_name",
    "tode_tableau",
    "tode_erk_stage",
    "tode_erk_combine",
    "tode_error_scale",
    "tode_row_norm",
    "tode_control",
    "tode_adapt_step",
    "tode_initial_step_a",
    "tode_initial_step_b",
    "tode_tolerance_scale",
    "tode_initial_step_a_norms",
    "tode_initial_step_b_norms",
    "tode_quartic_build",
    "tode_quartic_from_mid",
    "tode_cubic_build",
    "tode_poly_eval",
    "tode_poly_eval_masked",
    "tode_select_rows",
    "tode_loop_advance",
    "tode_loop_begin",
    "tode_count_initialized",
)

NORM_RMS, NORM_MAX = 0, 1
MAX_STAGES = 16
LOOP_ANY_RUNNING, LOOP_ANY_FAILURE, LOOP_N_TO_EVALUATE, LOOP_FLAG_WORDS = 0, 1, 2, 4


class Controller(C.Structure):
    """struct tode_controller"""

    _fields_ = [
        ("kind", C.c_int32),
        ("has_dt_min", C.c_int32),
        ("has_dt_max", C.c_int32),
        ("reserved", C.c_int32),
        ("atol", C.c_double),
        ("rtol", C.c_double),
        ("pcoeff", C.c_double),
        ("icoeff", C.c_double),
        ("dcoeff", C.c_double),
        ("safety", C.c_double),
        ("factor_min", C.c_double),
        ("factor_max", C.c_double),
        ("dt_min", C.c_double),
        ("dt_max", C.c_double),
    ]


class SolveArgs(C.Structure):
    """struct tode_solve_args"""

    _fields_ = [
        ("dtype", C.c_int32),
        ("method", C.c_int32),
        ("term", C.c_int32),
        ("n_features", C.c_int32),
        ("n_eval", C.c_int32),
        ("n_params", C.c_int32),
        ("batch", C.c_int64),
        ("max_steps", C.c_int64),
        ("iteration_cap", C.c_int64),
        ("term_scalars", C.c_double * 4),
        ("y0", C.c_void_p),
        ("t_start", C.c_void_p),
        ("t_end", C.c_void_p),
        ("t_start_stride", C.c_int64),
        ("t_end_stride", C.c_int64),
        ("t_eval", C.c_void_p),
        ("dt0", C.c_void_p),
        ("params", C.c_void_p),
        ("shared_params", C.c_void_p),
        ("n_shared_params", C.c_int64),
        ("ys", C.c_void_p),
        ("y_idle", C.c_void_p),
        ("pending", C.c_void_p),
        ("n_steps", C.c_void_p),
        ("n_accepted", C.c_void_p),
        ("n_initialized", C.c_void_p),
        ("status_last", C.c_void_p),
        ("status_idle", C.c_void_p),
        ("flags", C.c_void_p),
        ("record", C.c_void_p),
    ]


class SolveRecord(C.Structure):
    """struct tode_solve_record"""

    _fields_ = [("capacity", C.c_int64)] + [(n, C.c_void_p) for n in ("t", "dt", "y", "k0", "prev", "pprev", "running", "n_accepted")]


class SolveAdjoint(C.Structure):
    """struct tode_solve_adjoint"""

    _fields_ = [("grad_ys", C.c_void_p), ("points_by_iteration", C.c_void_p), ("iterations_sorted", C.c_void_p), ("iterations", C.c_int64), ("through_control", C.c_int32), ("through_start", C.c_int32),
                ("scratch", C.c_void_p), ("scratch_bytes", C.c_int64)] + [
        (n, C.c_void_p) for n in ("a_y", "a_k0", "a_t", "a_dt", "a_prev", "a_pprev", "g_params", "g_t_start", "g_t_end", "g_t_eval")
    ]  # fmt: skip


STEP_FLAG_STOPPED, STEP_FLAG_ITERATIONS, STEP_FLAG_ANY_RUNNING, STEP_FLAG_ANY_FAILURE, STEP_FLAG_WORDS = 0, 1, 2, 3, 4


class StepState(C.Structure):
    """struct tode_step_state"""

    _fields_ = [
        ("dtype", C.c_int32),
        ("time_dtype", C.c_int32),
        ("method", C.c_int32),
        ("n_features", C.c_int32),
        ("n_eval", C.c_int32),
        ("batch", C.c_int64),
        ("max_steps", C.c_int64),
        ("y0", C.c_void_p),
        ("t_start", C.c_void_p),
        ("t_end", C.c_void_p),
        ("t_eval", C.c_void_p),
        ("t", C.c_void_p),
        ("dt", C.c_void_p),
        ("y", C.c_void_p),
        ("k0", C.c_void_p),
        ("ratio_prev", C.c_void_p),
        ("ratio_pprev", C.c_void_p),
        ("running", C.c_void_p),
        ("cursor", C.c_void_p),
        ("n_steps", C.c_void_p),
        ("n_accepted", C.c_void_p),
        ("status", C.c_void_p),
        ("monotone", C.c_void_p),
        ("pending", C.c_void_p),
        ("ys", C.c_void_p),
        ("flags", C.c_void_p),
        ("ystage", C.c_void_p * 7),
        ("k", C.c_void_p * 7),
        ("tnode", C.c_void_p),
        ("host_flags", C.c_void_p),
        ("fixed_dt", C.c_void_p),
    ]


class StepAdjoint(C.Structure):
    """struct tode_step_adjoint"""

    _fields_ = [
        ("dtype", C.c_int32),
        ("time_dtype", C.c_int32),
        ("method", C.c_int32),
        ("n_features", C.c_int32),
        ("n_eval", C.c_int32),
        ("iteration", C.c_int32),
        ("through_control", C.c_int32),
        ("end_point", C.c_int32),
        ("batch", C.c_int64),
        ("t_start", C.c_void_p),
        ("t_end", C.c_void_p),
        ("t_eval", C.c_void_p),
        ("t", C.c_void_p),
        ("dt", C.c_void_p),
        ("y", C.c_void_p),
        ("ratio_prev", C.c_void_p),
        ("ratio_pprev", C.c_void_p),
        ("running", C.c_void_p),
        ("moved", C.c_void_p),
        ("running_next", C.c_void_p),
        ("k", C.c_void_p * 7),
        ("y1", C.c_void_p),
        ("fixed_dt", C.c_void_p),
        ("hit_iteration", C.c_void_p),
        ("grad_ys", C.c_void_p),
        ("a_t", C.c_void_p),
        ("a_dt", C.c_void_p),
        ("a_y", C.c_void_p),
        ("a_k0", C.c_void_p),
        ("a_prev", C.c_void_p),
        ("a_pprev", C.c_void_p),
        ("g_k", C.c_void_p * 7),
        ("g_y", C.c_void_p),
        ("g_y1", C.c_void_p),
        ("g_t", C.c_void_p),
        ("g_dt", C.c_void_p),
        ("g_prev", C.c_void_p),
        ("g_pprev", C.c_void_p),
        ("g_t_start", C.c_void_p),
        ("g_t_end", C.c_void_p),
        ("g_t_eval", C.c_void_p),
        ("g_fixed_dt", C.c_void_p),
    ]


class LoopArgs(C.Structure):
    """struct tode_loop_args"""

    _fields_ = [
        ("dtype", C.c_int32),
        ("n_features", C.c_int32),
        ("n_eval", C.c_int32),
        ("reserved", C.c_int32),
        ("batch", C.c_int64),
        ("max_steps", C.c_int64),
        ("t_start", C.c_void_p),
        ("t_end", C.c_void_p),
        ("t_eval", C.c_void_p),
        ("t", C.c_void_p),
        ("dt", C.c_void_p),
        ("y", C.c_void_p),
        ("running", C.c_void_p),
        ("y_new", C.c_void_p),
        ("accept", C.c_void_p),
        ("dt_next", C.c_void_p),
        ("method_status", C.c_void_p),
        ("controller_status", C.c_void_p),
        ("t_out", C.c_void_p),
        ("dt_out", C.c_void_p),
        ("y_out", C.c_void_p),
        ("running_out", C.c_void_p),
        ("to_update", C.c_void_p),
        ("status", C.c_void_p),
        ("n_steps", C.c_void_p),
        ("n_accepted", C.c_void_p),
        ("pending", C.c_void_p),
        ("to_evaluate", C.c_void_p),
        ("flags", C.c_void_p),
    ]


_lock = threading.Lock()
_lib = None


def load():
    """Returns the loaded library.  It is built first if the file is missing, and built again if it was made from
    other sources than the ones lying next to it (the library carries a hash of its sources): an edited kernel is
    never run through a stale binary.  Where the sources are absent (an installed copy) the file is taken as it is."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        from . import build

        if not os.path.exists(LIB_PATH):
            build.build_library(force=True)
        lib = C.CDLL(LIB_PATH)
        if os.path.isdir(build.CSRC):
            want = build.source_hash()
            lib.tode_source_hash.restype = C.c_char_p
            got = lib.tode_source_hash().decode() if hasattr(lib, "tode_source_hash") else ""
            if got != want:
                # (a loaded library cannot be replaced in this process: build, then load the new file under a new name)
                import shutil
                import tempfile
                import warnings

                warnings.warn("libtorchode_amd.so was built from other sources than those in torchode_amd/csrc: rebuilding it")
                build.build_library(force=True)
                fresh = os.path.join(tempfile.mkdtemp(prefix="torchode_amd_"), "libtorchode_amd.so")
                shutil.copy(LIB_PATH, fresh)
                lib = C.CDLL(fresh)
                lib.tode_source_hash.restype = C.c_char_p
                if lib.tode_source_hash().decode() != want:
                    raise RuntimeError("libtorchode_amd.so does not match its sources even after a rebuild")
        lib.tode_abi_version.restype = C.c_int
        lib.tode_last_error.restype = C.c_char_p
        lib.tode_solve_builtin.restype = C.c_int
        lib.tode_solve_builtin.argtypes = [C.POINTER(SolveArgs), C.POINTER(Controller), C.c_void_p]
        lib.tode_solve_builtin_fast.restype = C.c_int
        lib.tode_solve_builtin_fast.argtypes = [C.POINTER(SolveArgs), C.POINTER(Controller)] + [C.c_void_p] * 5
        lib.tode_select_end_point.restype = C.c_int
        lib.tode_select_end_point.argtypes = [C.c_int64, C.c_int32, C.c_int32, C.c_int64, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]
        lib.tode_mlp_pack_weights.restype = C.c_int
        lib.tode_mlp_pack_weights.argtypes = [C.c_void_p, C.c_int64, C.c_int32, C.c_void_p, C.c_void_p]
        lib.tode_mlp_pack_weights_for.restype = C.c_int
        lib.tode_mlp_pack_weights_for.argtypes = [C.c_void_p, C.c_int64, C.c_int32, C.c_int32, C.c_void_p, C.c_void_p]
        lib.tode_solve_builtin_fast_static.restype = C.c_int
        lib.tode_solve_builtin_fast_static.argtypes = [C.POINTER(SolveArgs), C.POINTER(Controller)] + [C.c_void_p] * 6
        lib.tode_solve_builtin_fast_sync.restype = C.c_int
        lib.tode_solve_builtin_fast_sync.argtypes = [C.POINTER(SolveArgs), C.POINTER(Controller)] + [C.c_void_p] * 5 + [C.POINTER(C.c_int32)]
        lib.tode_solve_workspace_bytes.restype = C.c_int64
        lib.tode_solve_workspace_bytes.argtypes = [C.POINTER(SolveArgs)]
        lib.tode_solve_builtin_auto.restype = C.c_int
        lib.tode_solve_builtin_auto.argtypes = [C.POINTER(SolveArgs), C.POINTER(Controller)] + [C.c_void_p] * 5 + [C.c_int64, C.c_int32, C.c_void_p, C.POINTER(C.c_int64)]
        lib.tode_solve_backward_scratch_bytes.restype = C.c_int64
        lib.tode_solve_backward_scratch_bytes.argtypes = [C.POINTER(SolveArgs)]
        lib.tode_solve_builtin_backward.restype = C.c_int
        lib.tode_solve_builtin_backward.argtypes = [C.POINTER(SolveArgs), C.POINTER(Controller), C.POINTER(SolveAdjoint), C.c_void_p]
        lib.tode_step_begin.restype = C.c_int
        lib.tode_step_begin.argtypes = [C.POINTER(StepState), C.POINTER(Controller), C.c_void_p, C.c_int, C.c_void_p]
        lib.tode_step_stage.restype = C.c_int
        lib.tode_step_stage.argtypes = [C.POINTER(StepState), C.POINTER(Controller), C.c_int, C.c_void_p]
        lib.tode_step_finish_backward.restype = C.c_int
        lib.tode_step_finish_backward.argtypes = [C.POINTER(StepAdjoint), C.POINTER(Controller), C.c_void_p]
        lib.tode_step_stage_backward.restype = C.c_int
        lib.tode_step_stage_backward.argtypes = [C.POINTER(StepAdjoint), C.POINTER(Controller), C.c_int, C.c_void_p, C.c_void_p, C.c_void_p]
        lib.tode_step_finish.restype = C.c_int
        lib.tode_step_finish.argtypes = [C.POINTER(StepState), C.POINTER(Controller), C.c_void_p]
        lib.tode_step_stats.restype = C.c_int
        lib.tode_step_stats.argtypes = [C.POINTER(StepState)] + [C.c_void_p] * 5
        lib.tode_finalize_stats.restype = C.c_int
        lib.tode_finalize_stats.argtypes = [C.c_int64, C.c_int64] + [C.c_void_p] * 9 + [C.c_int32] * 3 + [C.c_void_p] * 3
        lib.tode_set_fast_kernel_variant.restype = C.c_int
        lib.tode_set_fast_kernel_variant.argtypes = [C.c_int]
        lib.tode_set_kernel_timing.restype = C.c_int
        lib.tode_set_kernel_timing.argtypes = [C.c_int]
        lib.tode_last_solve_kernel_ms.restype = C.c_int
        lib.tode_last_solve_kernel_name.restype = C.c_char_p
        lib.tode_last_solve_kernel_name.argtypes = []
        lib.tode_last_solve_kernel_ms.argtypes = [C.POINTER(C.c_float)]
        V, I32, I64, D = C.c_void_p, C.c_int32, C.c_int64, C.c_double
        DP, CP = C.POINTER(C.c_double), C.POINTER(Controller)
        for name, argtypes in {
            "tode_tableau": [I32, DP, DP, DP, DP, C.POINTER(I32)],
            "tode_erk_stage": [I32, I64, I32, I32, DP, D] + [V] * 7,
            "tode_erk_combine": [I32, I64, I32, I32, DP] + [V] * 5,
            "tode_error_scale": [I32, I64, I32, D, D] + [V] * 5,
            "tode_row_norm": [I32, I32, I64, I32] + [V] * 3,
            "tode_control": [I32, CP, I32, I64] + [V] * 11,
            "tode_adapt_step": [I32, CP, I32, I32, I64, I32] + [V] * 13,
            "tode_initial_step_a": [I32, I32, I64, I32, D, D] + [V] * 8,
            "tode_initial_step_b": [I32, I32, I32, I32, I64, I32, D, D] + [V] * 8,
            "tode_tolerance_scale": [I32, I64, I32, D, D] + [V] * 4,
            "tode_initial_step_a_norms": [I32, I64, I32] + [V] * 10,
            "tode_initial_step_b_norms": [I32, I32, I32, I64] + [V] * 7,
            "tode_quartic_build": [I32, I32, I64, I32] + [V] * 6,
            "tode_quartic_from_mid": [I32, I64, I32] + [V] * 8,
            "tode_cubic_build": [I32, I64, I32] + [V] * 7,
            "tode_poly_eval": [I32, I32, I32, I64, I32, I64] + [V] * 7,
            "tode_poly_eval_masked": [I32, I32, I32, I64, I32, I32] + [V] * 7,
            "tode_select_rows": [I32, I64, I32] + [V] * 5,
            "tode_loop_advance": [C.POINTER(LoopArgs), V],
            "tode_loop_begin": [I32, I64, I32, I32] + [V] * 9,
            "tode_count_initialized": [I64, I32, V, V, V],
        }.items():
            fn = getattr(lib, name)
            fn.restype, fn.argtypes = C.c_int, argtypes
        got = lib.tode_abi_version()
        if got != ABI_VERSION:
            raise RuntimeError(f"libtorchode_amd.so has ABI version {got}, the Python package expects {ABI_VERSION}")
        _lib = lib
        return _lib


def check(rc: int, what: str):
    if rc != 0:
        msg = load().tode_last_error().decode("utf-8", "replace")
        raise RuntimeError(f"{what} failed with code {rc}: {msg}")


def dtype_code(data_dtype, time_dtype=None) -> int:
    """``dtype`` argument of the operator entry points (TODE_DTYPES in the header)."""
    if data_dtype not in DTYPES or (time_dtype is not None and time_dtype not in DTYPES):
        raise NotImplementedError(f"the kernels are built for float32 and float64 (got data {data_dtype}, time {time_dtype})")
    if time_dtype is None or time_dtype == data_dtype:
        return DTYPES[data_dtype]
    return 0x100 | DTYPES[data_dtype] | (DTYPES[time_dtype] << 4)


def ptr(t):
    return None if t is None else C.c_void_p(t.data_ptr())


def require_device(*tensors):
    """The kernels run on a HIP device only; anything else is an error, never a fallback."""
    for t in tensors:
        if t is not None and t.device.type != "cuda":
            raise RuntimeError(
                "torchode_amd runs on an AMD GPU (HIP device) only; got a tensor on "
                f"'{t.device}'. There is no CPU implementation to fall back to."
            )


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def stream_of(t) -> C.c_void_p:
    """PyTorch's current stream on the tensor's device, as the handle the C ABI takes."""
    if _raw_stream is not None:  # (the handle without a Stream object around it: 0.3 instead of 3 microseconds)
        return C.c_void_p(_raw_stream(t.device.index if t.device.index is not None else torch.cuda.current_device()))
    return C.c_void_p(torch.cuda.current_stream(t.device).cuda_stream)


def set_kernel_timing(enable: bool):
    """Record HIP events around the solve kernel of subsequent solves made by this thread."""
    check(load().tode_set_kernel_timing(int(enable)), "tode_set_kernel_timing")


def last_solve_kernel_ms() -> float:
    """Duration of the most recent solve kernel launched by this thread (waits for it)."""
    out = C.c_float(0.0)
    check(load().tode_last_solve_kernel_ms(C.byref(out)), "tode_last_solve_kernel_ms")
    return out.value


def last_solve_kernel_name() -> str:
    """Name of the solve kernel most recently launched by this thread (as a profiler shows it)."""
    return load().tode_last_solve_kernel_name().decode()


def set_fast_kernel_variant(variant: int):
    """0: automatic, 1: one wavefront per 64 samples, 2: stepper + evaluator wavefronts."""
    check(load().tode_set_fast_kernel_variant(int(variant)), "tode_set_fast_kernel_variant")
