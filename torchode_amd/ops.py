"""``torch.ops.torchode_amd``: the whole-solve entry point of the C ABI as PyTorch operators.

The library's own eager path calls the C ABI through ``ctypes`` (``_lib.py``; fewer microseconds per
call than the dispatcher).  The operators here are the same entry points for programs that PyTorch
captures: ``torch.compile(solver.solve)`` with a built-in term records the whole solve as one node,
``torchode_amd::solve_builtin``, instead of breaking the graph at a foreign function call.  The
operators are registered by ``libtorchode_amd_ops.so`` (``csrc/tode_torch_ops.cpp``, built by
``torchode_amd.build`` next to ``libtorchode_amd.so``), for the GPU only: there is no CPU
implementation, and a call with CPU tensors fails in the dispatcher.  Shapes and dtypes of the
results for tracing come from the functions registered below.

Reference: the loop these replace is ``AutoDiffAdjoint.solve`` (adjoints.py:42-311); the reference's
own route to a compiled solve is ``torch.compile`` of that loop (docs/jit.ipynb).
"""
import os
import threading
from typing import Optional, Sequence

import torch

from . import _lib, build

_lock = threading.Lock()
_loaded = False


def load() -> None:
    """Loads the operator library (after the library it calls into) and registers the tracing rules."""
    if not _loaded:  # (read without the lock: a tracer that runs through here sees one global and no lock)
        _load_once()


@torch.compiler.disable
def _load_once() -> None:
    global _loaded
    with _lock:
        if _loaded:
            return
        _lib.load()
        if not os.path.exists(build.OPS_LIB):
            build.link_ops_library()
        torch.ops.load_library(build.OPS_LIB)

        @torch.library.register_fake("torchode_amd::solve_builtin")
        def _(y0, t_start, t_end, t_eval, dt0, params, shared_params, method, term, term_scalars, controller_kind, control, max_steps, allow_one_kernel):
            B, F = y0.shape
            E = 1 if t_eval is None else max(t_eval.shape[1], 1)
            stat = lambda: y0.new_empty((B,), dtype=torch.long)
            return y0.new_empty((B, E, F)), stat(), stat(), stat(), stat(), torch.empty((), dtype=torch.long, device="cpu")

        @torch.library.register_fake("torchode_amd::mlp_pack_weights")
        def _(raw, matrix_inputs, n_features=64):
            return raw.new_empty((_lib.MLP_PACKED_SIZE["bfloat16" if matrix_inputs == _lib.MLP_INPUTS["bfloat16"] else "float32"],))

        _loaded = True


def solve_builtin(
    y0: torch.Tensor,
    t_start: torch.Tensor,
    t_end: torch.Tensor,
    t_eval: Optional[torch.Tensor],
    dt0: Optional[torch.Tensor],
    params: Optional[torch.Tensor],
    shared_params: Optional[torch.Tensor],
    method: int,
    term: int,
    term_scalars: Sequence[float],
    controller_kind: int,
    control: Sequence[float],
    max_steps: Optional[int] = None,
    allow_one_kernel: bool = True,
):
    """``(ys, n_steps, n_accepted, n_initialized, status, iterations)`` of one whole solve with a built-in term
    (``tode_solve_builtin_auto``).  ``iterations`` is an int64 scalar on the CPU: the loop iterations, from which
    ``stats["n_f_evals"]`` follows."""
    load()
    return torch.ops.torchode_amd.solve_builtin(
        y0, t_start, t_end, t_eval, dt0, params, shared_params, method, term, list(term_scalars), controller_kind, list(control),
        -1 if max_steps is None else int(max_steps), allow_one_kernel,
    )  # fmt: skip


def mlp_pack_weights(raw: torch.Tensor, matrix_inputs: int, n_features: int = 64) -> torch.Tensor:
    load()
    return torch.ops.torchode_amd.mlp_pack_weights(raw, matrix_inputs, n_features)
