"""Norms. ``RMSNorm`` follows nanovllm/layers/layernorm.py:16-40."""
from __future__ import annotations

import torch

from ..native import ops
from .base import NORMS, ParamSpec, Part


@NORMS.register("rmsnorm")
class RMSNorm(Part):
    """y = x / sqrt(mean(x^2) + eps) * weight; with a residual the sum is normed
    and carried on (layernorm.py:28-40)."""

    def __init__(self, size: int, eps: float, residual_float32: bool = True):
        """``residual_float32`` (an engine option, offered to every part when a model is built): True: the residual
        stream is carried in float32 whatever the rows' element type, so the sum goes from layer to layer
        unrounded. False: it is carried in the rows' element type, rounded after every addition, as the
        reference carries it (layernorm.py:34-40; the norm itself still takes the unrounded float sum)."""
        self.size = size
        self.eps = eps
        self.residual_float32 = bool(residual_float32)
        self.weight = None

    def param_specs(self):
        return {"weight": ParamSpec((self.size,), init="norm", keeps_float32=True)}

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return ops.rmsnorm(x, self.weight, self.eps)

    def forward_start(self, x: torch.Tensor):
        """The first norm of a model: returns (norm(x), x as the residual that later norms add to)."""
        return ops.rmsnorm(x, self.weight, self.eps, start_residual=True, residual_float32=self.residual_float32)

    def forward_add(self, x: torch.Tensor, residual: torch.Tensor):
        """Returns (norm(x + residual), x + residual); ``residual`` is updated in place."""
        y = ops.rmsnorm(x, self.weight, self.eps, residual=residual)
        return y, residual
