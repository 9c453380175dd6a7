"""Norms. ``RMSNorm`` follows nanovllm/layers/layernorm.py:16-40."""
from __future__ import annotations

import torch

from ..native import ops
from .base import NORMS, ParamSpec, Part


@NORMS.register("rmsnorm")
class RMSNorm(Part):
    """y = x / sqrt(mean(x^2) + eps) * weight; with a residual the sum is normed
    and carried on (layernorm.py:28-40)."""

    def __init__(self, size: int, eps: float):
        self.size = size
        self.eps = eps
        self.weight = None

    def param_specs(self):
        return {"weight": ParamSpec((self.size,), init="norm", keeps_float32=True)}

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return ops.rmsnorm(x, self.weight, self.eps)

    def forward_start(self, x: torch.Tensor):
        """The first norm of a model: returns (norm(x), x as the residual that later norms add to).
        The residual is kept in float32 whatever the rows' element type, so the sum is
        carried from layer to layer without rounding."""
        return ops.rmsnorm(x, self.weight, self.eps, start_residual=True)

    def forward_add(self, x: torch.Tensor, residual: torch.Tensor):
        """Returns (norm(x + residual), x + residual); ``residual`` is updated in place."""
        y = ops.rmsnorm(x, self.weight, self.eps, residual=residual)
        return y, residual
