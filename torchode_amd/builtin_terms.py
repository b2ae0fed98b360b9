"""Right-hand sides that the persistent whole-solve kernels know natively.

Each class is an ordinary ``f(t, y)`` torch module -- it can be wrapped in
``ODETerm`` and used with any solver path -- and additionally carries a
``builtin_kind`` tag plus a per-sample parameter table, which lets
``AutoDiffAdjoint.solve`` run the entire solve for it inside one HIP kernel.
``forward`` spells out the op order that the kernels reproduce (each torch op
rounds on its own; the kernels are compiled without floating point contraction).
"""
import torch
import torch.nn as nn

# numeric tags shared with the C ABI (include/torchode_amd.h, TODE_TERM_*)
TERM_LINEAR_DECAY = 0
TERM_VAN_DER_POL = 1
TERM_LORENZ63 = 2


class BuiltinTerm(nn.Module):
    builtin_kind: int = -1
    n_features: int = 0

    def builtin_params(self) -> torch.Tensor:
        """Per-sample parameters as a contiguous ``[B, P]`` tensor in the data dtype."""
        raise NotImplementedError


class LinearDecay(BuiltinTerm):
    """``dy/dt = (-k) * y`` with one rate per sample and feature, ``k`` of shape ``[B, F]``."""

    builtin_kind = TERM_LINEAR_DECAY

    def __init__(self, k: torch.Tensor):
        super().__init__()
        assert k.ndim == 2
        self.register_buffer("k", k)
        self.n_features = k.shape[1]

    def forward(self, t, y):
        return (-self.k) * y

    def builtin_params(self):
        return self.k.contiguous()


class VanDerPol(BuiltinTerm):
    """``y = (x, v)``, ``dx = v``, ``dv = ((mu * (1 - (x * x))) * v) - x``; ``mu`` of shape ``[B]``."""

    builtin_kind = TERM_VAN_DER_POL
    n_features = 2

    def __init__(self, mu: torch.Tensor):
        super().__init__()
        assert mu.ndim == 1
        self.register_buffer("mu", mu)

    def forward(self, t, y):
        x, v = y[:, 0], y[:, 1]
        dv = ((self.mu * (1 - (x * x))) * v) - x
        return torch.stack((v, dv), dim=1)

    def builtin_params(self):
        return self.mu.reshape(-1, 1).contiguous()


class Lorenz63(BuiltinTerm):
    """Lorenz-63 with per-sample ``rho`` (shape ``[B]``) and scalar ``sigma``, ``beta``:
    ``dx = sigma*(y-x)``, ``dy = (x*(rho-z)) - y``, ``dz = (x*y) - (beta*z)``."""

    builtin_kind = TERM_LORENZ63
    n_features = 3

    def __init__(self, rho: torch.Tensor, sigma: float = 10.0, beta: float = 8.0 / 3.0):
        super().__init__()
        assert rho.ndim == 1
        self.register_buffer("rho", rho)
        self.sigma = float(sigma)
        self.beta = float(beta)

    def forward(self, t, y):
        x, yy, z = y[:, 0], y[:, 1], y[:, 2]
        dx = self.sigma * (yy - x)
        dy = (x * (self.rho - z)) - yy
        dz = (x * yy) - (self.beta * z)
        return torch.stack((dx, dy, dz), dim=1)

    def builtin_params(self):
        return self.rho.reshape(-1, 1).contiguous()

    def builtin_scalars(self):
        return (self.sigma, self.beta)
