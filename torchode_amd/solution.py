"""What a solve returns (reference torchode/solution.py:6-23)."""
from typing import Any, Dict

import torch


class Solution:
    """``ts [B,E]``, ``ys [B,E,F]``, ``stats`` (``n_f_evals`` on the CPU, ``n_steps``,
    ``n_accepted``, ``n_initialized`` on the data device, all int64 ``[B]``) and the
    per-sample ``status`` codes.  Rows of ``ys`` at or beyond ``n_initialized`` hold
    unspecified values after an early stop."""

    FIELDS = ("ts", "ys", "stats", "status")

    def __init__(self, ts: torch.Tensor, ys: torch.Tensor, stats: Dict[str, Any], status: torch.Tensor):
        self.ts, self.ys, self.stats, self.status = ts, ys, stats, status

    def __repr__(self):
        return "Solution(" + ", ".join(f"{name}={getattr(self, name)}" for name in self.FIELDS) + ")"
