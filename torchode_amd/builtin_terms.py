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
TERM_REACTION_DIFFUSION = 3
TERM_MLP = 4


class BuiltinTerm(nn.Module):
    builtin_kind: int = -1
    n_features: int = 0

    def builtin_params(self) -> torch.Tensor:
        """Per-sample parameters as a contiguous ``[B, P]`` tensor in the data dtype."""
        raise NotImplementedError

    def hold(self, name: str, tensor: torch.Tensor) -> None:
        """Keeps a tensor of the term: an ``nn.Parameter`` as a parameter (so that optimizers and the backsolve adjoints,
        which differentiate with respect to ``term.parameters()``, find it), any other tensor as a buffer."""
        if isinstance(tensor, nn.Parameter):
            self.register_parameter(name, tensor)
        else:
            self.register_buffer(name, tensor)


class LinearDecay(BuiltinTerm):
    """``dy/dt = (-k) * y`` with one rate per sample and feature, ``k`` of shape ``[B, F]``."""

    builtin_kind = TERM_LINEAR_DECAY

    def __init__(self, k: torch.Tensor):
        super().__init__()
        assert k.ndim == 2
        self.hold("k", k)
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
        self.hold("mu", mu)

    def forward(self, t, y):
        x, v = y[:, 0], y[:, 1]
        dv = ((self.mu * (1 - (x * x))) * v) - x
        return torch.stack((v, dv), dim=1)

    def builtin_params(self):
        if torch.compiler.is_compiling():  # (the cache below keys on the tensor's version counter, which a tracer cannot read)
            return self.mu.reshape(-1, 1)
        mu = self._buffers.get("mu")  # (a dictionary read; `self.mu` goes through nn.Module.__getattr__)
        if mu is None:
            mu = self.mu
        cached = self.__dict__.get("_params_view")
        if cached is None or cached[0] is not mu or cached[1] != mu._version:
            cached = self.__dict__["_params_view"] = (mu, mu._version, mu.reshape(-1, 1).contiguous())
        return cached[2]


class Lorenz63(BuiltinTerm):
    """Lorenz-63 with per-sample ``rho`` (shape ``[B]``) and scalar ``sigma``, ``beta``:
    ``dx = sigma*(y-x)``, ``dy = (x*(rho-z)) - y``, ``dz = (x*y) - (beta*z)``."""

    builtin_kind = TERM_LORENZ63
    n_features = 3

    def __init__(self, rho: torch.Tensor, sigma: float = 10.0, beta: float = 8.0 / 3.0):
        super().__init__()
        assert rho.ndim == 1
        self.hold("rho", rho)
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


class ReactionDiffusion(BuiltinTerm):
    """Fisher-KPP reaction-diffusion on a periodic ``n x n`` grid with unit spacing, one
    diffusivity per sample (``D`` of shape ``[B]``); the state is the flattened grid, ``F = n*n``:
    ``du/dt = D * lap(u) + u * (1 - u)`` with the five-point Laplacian summed as
    ``(((up + down) + left) + right) - 4u``."""

    builtin_kind = TERM_REACTION_DIFFUSION

    def __init__(self, D: torch.Tensor, n: int = 64):
        super().__init__()
        assert D.ndim == 1
        self.hold("D", D)
        self.n = int(n)
        self.n_features = self.n * self.n

    def forward(self, t, y):
        u = y.view(y.shape[0], self.n, self.n)
        lap = (((torch.roll(u, 1, 1) + torch.roll(u, -1, 1)) + torch.roll(u, 1, 2)) + torch.roll(u, -1, 2)) - (4 * u)
        return (self.D[:, None, None] * lap + u * (1 - u)).flatten(1)

    def builtin_params(self):
        return self.D.reshape(-1, 1).contiguous()


class MLPField(BuiltinTerm):
    """Time-dependent two-layer perceptron shared by the whole batch:
    ``f(t, y) = tanh(cat([y, t], 1) @ W1.T + b1) @ W2.T + b2`` with ``W1 [H, F+1]``, ``W2 [F, H]``.

    ``matrix_inputs="bfloat16"`` is a reduced-precision variant of the function itself: both matrix
    products take their two operands rounded to bfloat16 (sums, biases and tanh stay in the working
    precision), which is what the matrix cores do at eight times the float32 rate."""

    builtin_kind = TERM_MLP

    def __init__(self, W1: torch.Tensor, b1: torch.Tensor, W2: torch.Tensor, b2: torch.Tensor, matrix_inputs: str = "float32"):
        super().__init__()
        assert W1.ndim == 2 and W2.ndim == 2 and W1.shape[0] == W2.shape[1] and W1.shape[1] == W2.shape[0] + 1
        assert matrix_inputs in ("float32", "bfloat16")
        for name, w in (("W1", W1), ("b1", b1), ("W2", W2), ("b2", b2)):
            self.hold(name, w)
        self.n_features = W2.shape[0]
        self.matrix_inputs = matrix_inputs

    def forward(self, t, y):
        x = torch.cat([y, t[..., None]], -1)  # (also one sample at a time, as the backsolve adjoint's vmap calls it)
        if self.matrix_inputs == "bfloat16":
            rounded = lambda z: z.to(torch.bfloat16).to(z.dtype)
            h = torch.tanh(rounded(x) @ rounded(self.W1).T + self.b1)
            return rounded(h) @ rounded(self.W2).T + self.b2
        h = torch.tanh(x @ self.W1.T + self.b1)
        return h @ self.W2.T + self.b2

    def builtin_params(self):
        return torch.empty((0, 0), dtype=self.W1.dtype, device=self.W1.device)

    def builtin_shared(self) -> torch.Tensor:
        """W1 | b1 | W2 | b2, row-major and concatenated."""
        return torch.cat([w.reshape(-1) for w in (self.W1, self.b1, self.W2, self.b2)]).contiguous()

    def builtin_packed(self, device, dtype) -> torch.Tensor:
        """The weights in the order the whole-solve kernel loads them into registers (a device
        tensor).  Packed once, and again whenever a weight tensor has been replaced or written
        in place."""
        from . import _lib

        weights = (self.W1, self.b1, self.W2, self.b2)
        key = (tuple((w.data_ptr(), w._version) for w in weights), device, dtype, self.matrix_inputs)
        if getattr(self, "_packed_key", None) != key:
            raw = self.builtin_shared().to(device=device, dtype=dtype)
            packed = torch.empty(_lib.MLP_PACKED_SIZE[self.matrix_inputs], dtype=dtype, device=device)
            rc = _lib.load().tode_mlp_pack_weights_for(
                _lib.ptr(raw), raw.numel(), self.W2.shape[0], _lib.MLP_INPUTS[self.matrix_inputs], _lib.ptr(packed),
                _lib.stream_of(raw),
            )
            _lib.check(rc, "tode_mlp_pack_weights_for")
            self._packed, self._packed_key = packed, key
        return self._packed
