"""Norms. ``RMSNorm`` follows nanovllm/layers/layernorm.py:16-40."""
from __future__ import annotations

import torch

from ..native import ops
from .base import NORMS, ParamSpec, Part


@NORMS.register("rmsnorm")
class RMSNorm(Part):
    """y = x / sqrt(mean(x^2) + eps) * weight; with a residual the sum is normed
    and carried on (layernorm.py:28-40)."""

    takes_summed = True           # ``forward_add`` takes an ``ops.Summed`` (a sum that a product has made already)
    defers_to_products = True     # ``forward_add(..., deferred=True)`` may return an ``ops.Normed``

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

    def forward_start(self, x: torch.Tensor):
        """The first norm of a model: returns (norm(x), x as the residual that later norms add to)."""
        return ops.rmsnorm(x, self.weight, self.eps, start_residual=True, residual_float32=self.residual_float32)

    def forward(self, x) -> torch.Tensor:
        return ops.rmsnorm(ops.dense(x), self.weight, self.eps)

    def add_to(self, residual: torch.Tensor, reader=None) -> ops.AddTo:
        """What the part before this norm is handed so that its last product can make the addition to ``residual``
        and this norm's product with its weight (``forward_add`` then gets an ``ops.Summed``). ``reader``: the part
        that reads this norm, if it says what its first product is (``first_product()``)."""
        first = getattr(reader, "first_product", None)
        return ops.AddTo(residual, self.weight, self.eps, first() if first is not None else None)

    def forward_add(self, x, residual: torch.Tensor, deferred: bool = False):
        """Returns (norm(x + residual), x + residual); ``residual`` is updated in place. ``x`` may be the
        ``ops.Summed`` that a product made from this norm's ``add_to``: the sum is in ``residual`` already, and what
        is left of the norm is the scaling of the rows. ``deferred``: the caller's next step is a product, which
        scales its rows itself; it then gets an ``ops.Normed`` in place of a tensor."""
        if isinstance(x, ops.Summed):
            if x.norm_weight is not self.weight or x.residual is not residual:
                raise ValueError("a sum that a product made for another norm, or into another residual stream")
            normed = ops.Normed(x)
            return (normed if deferred else normed.tensor()), residual
        y = ops.rmsnorm(x, self.weight, self.eps, residual=residual)
        return y, residual
