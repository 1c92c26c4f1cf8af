"""RMSNorm part: ``x * rsqrt(mean(x^2) + eps) * weight`` in float32
(reference: ``src/mini_engine/model.py:59-69``; the weight multiplies directly, eps inside the root)."""

from __future__ import annotations

import torch

from ..ops import kernels as K
from ..weights.loader import TensorWant
from .base import NORMS, Norm


class RMSNorm(Norm):
    graph_safe = True

    def __init__(self, spec, dtype, device):
        super().__init__(spec, dtype, device)
        self.eps = float(spec.eps)
        self.dim = int(spec.dim)
        self.weight = torch.ones(self.dim, dtype=torch.float32, device=device)

    def weight_wants(self, name: str) -> dict[str, TensorWant]:
        return {name: TensorWant((self.dim,), "vector")}

    def load(self, tensors, name: str) -> None:
        self.weight = tensors[name]

    def as_fused(self):
        return self.weight, self.eps

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return K.add_rmsnorm(x, None, self.weight, self.eps, self.dtype, write_x=False)

    def __call__(self, x: torch.Tensor) -> torch.Tensor:
        """Norm of activations [..., dim] in the compute dtype (no residual involved)."""
        return K.rmsnorm(x, self.weight, self.eps)


NORMS.register("rmsnorm", RMSNorm)
