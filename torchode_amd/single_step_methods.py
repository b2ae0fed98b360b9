"""Explicit Runge-Kutta pairs (mirror torchode/single_step_methods/dopri5.py, tsit5.py).

``Dopri5`` and ``Tsit5`` are 7-stage FSAL pairs of convergence order 5 with a
quartic dense output.  Their coefficients live in the device code
(csrc/tode_math.h); these classes carry the identity of the method and the
optional fixed term.
"""
from typing import Optional

import torch.nn as nn

from . import _lib
from .terms import ODETerm


class ExplicitRungeKutta(nn.Module):
    method_id = -1

    def __init__(self, term: Optional[ODETerm] = None):
        super().__init__()
        self.term = term

    def convergence_order(self) -> int:
        return 5


class Dopri5(ExplicitRungeKutta):
    """Dormand-Prince 5(4)."""

    method_id = _lib.DOPRI5


class Tsit5(ExplicitRungeKutta):
    """Tsitouras 5(4)."""

    method_id = _lib.TSIT5
