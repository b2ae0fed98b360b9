"""Adaptive step size controllers (mirror torchode/step_size_controllers.py:260-835).

The classes keep the reference's constructor signatures and protocol methods.
Their arithmetic runs in HIP kernels: inside the persistent whole-solve kernel
when ``AutoDiffAdjoint`` recognises the whole configuration, and in the per-step
kernels otherwise.
"""
from math import sqrt
from typing import Callable, Optional

import torch
import torch.nn as nn

from . import _lib
from .terms import ODETerm


def rms_norm(y: torch.Tensor) -> torch.Tensor:
    """Root mean square norm over the feature dimension (Hairer, Norsett & Wanner I, eq. II.4.11;
    reference step_size_controllers.py:170-181).  Passing this function as ``norm`` (the default)
    selects the fused kernels, which compute the same quantity on the device."""
    return torch.linalg.vector_norm(y / sqrt(y.shape[1]), ord=2, dim=1)


def max_norm(y: torch.Tensor) -> torch.Tensor:
    """Maximum norm over the feature dimension (reference step_size_controllers.py:184-186)."""
    return torch.linalg.vector_norm(y, dim=1, ord=torch.inf)


class _AdaptiveController(nn.Module):
    _kind = -1

    def __init__(self, atol, rtol, pcoeff, icoeff, dcoeff, term, norm, dt_min, dt_max, safety, factor_min, factor_max):
        super().__init__()
        # float32 buffers, as in the reference: the tolerances take effect float32-rounded
        # even in a float64 solve
        self.register_buffer("atol", torch.tensor(atol))
        self.register_buffer("rtol", torch.tensor(rtol))
        self.term = term
        self.norm = norm
        self.dt_min = dt_min
        self.dt_max = dt_max
        self.pcoeff = pcoeff
        self.icoeff = icoeff
        self.dcoeff = dcoeff
        self.safety = safety
        self.factor_min = factor_min
        self.factor_max = factor_max
        self._atol_f = float(torch.tensor(atol))
        self._rtol_f = float(torch.tensor(rtol))

    @property
    def fusable(self) -> bool:
        """True when the device kernels implement this controller exactly (RMS norm)."""
        return self.norm is rms_norm

    def c_struct(self) -> "_lib.Controller":
        """Parameters in the layout of ``struct tode_controller``."""
        return _lib.Controller(
            self._kind,
            self.dt_min is not None,
            self.dt_max is not None,
            0,
            self._atol_f,
            self._rtol_f,
            float(self.pcoeff),
            float(self.icoeff),
            float(self.dcoeff),
            float(self.safety),
            float(self.factor_min),
            float(self.factor_max),
            float(self.dt_min or 0.0),
            float(self.dt_max or 0.0),
        )


class IntegralController(_AdaptiveController):
    """Scales the step by ``safety * ratio**(-1/order)`` clipped to ``[factor_min, factor_max]``
    (reference step_size_controllers.py:260-294)."""

    _kind = _lib.CTRL_INTEGRAL

    def __init__(
        self,
        atol: float,
        rtol: float,
        *,
        term: Optional[ODETerm] = None,
        norm: Callable = rms_norm,
        dt_min: Optional[float] = None,
        dt_max: Optional[float] = None,
        safety: float = 0.9,
        factor_min: float = 0.2,
        factor_max: float = 10.0,
    ):
        super().__init__(atol, rtol, 0.0, 1.0, 0.0, term, norm, dt_min, dt_max, safety, factor_min, factor_max)


class PIDController(_AdaptiveController):
    """PID step size control after Soederlind (2003), eq. (34), with the coefficients divided by
    the method order (reference step_size_controllers.py:554-620)."""

    _kind = _lib.CTRL_PID

    def __init__(
        self,
        atol: float,
        rtol: float,
        pcoeff: float,
        icoeff: float,
        dcoeff: float,
        *,
        term: Optional[ODETerm] = None,
        norm: Callable = rms_norm,
        dt_min: Optional[float] = None,
        dt_max: Optional[float] = None,
        safety: float = 0.9,
        factor_min: float = 0.2,
        factor_max: float = 10.0,
    ):
        super().__init__(atol, rtol, pcoeff, icoeff, dcoeff, term, norm, dt_min, dt_max, safety, factor_min, factor_max)
