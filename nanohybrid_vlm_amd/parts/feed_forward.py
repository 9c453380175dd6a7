"""Feed-forward parts. ``SwiGLU`` follows nanovllm/models/qwen3.py:91-117."""
from __future__ import annotations

import torch

from ..native import ops
from .base import FEED_FORWARDS, ParamSpec, Part


@FEED_FORWARDS.register("swiglu")
class SwiGLU(Part):
    """down(silu(gate(x)) * up(x)); gate and up are one packed matrix whose first
    ``intermediate_size`` rows are the gate (nanovllm/layers/linear.py:102-108,
    nanovllm/layers/activation.py:10-11)."""

    def __init__(self, hidden_size: int, intermediate_size: int):
        self.hidden_size = hidden_size
        self.intermediate_size = intermediate_size
        self.gate_up_weight = None
        self.down_weight = None

    def param_specs(self):
        return {
            "gate_up.weight": ParamSpec((2 * self.intermediate_size, self.hidden_size)),
            "down.weight": ParamSpec((self.hidden_size, self.intermediate_size)),
        }

    takes_deferred_norm = True    # x goes straight into a product, which can norm it
    adds_to_residual = True       # the down projection can make the addition to the residual stream

    def first_product(self):
        """(weight, gated) of the product that x goes into."""
        return self.gate_up_weight, True

    def forward(self, x, step, add_to=None):
        return ops.linear(ops.gated_linear(x, self.gate_up_weight), self.down_weight, add_to=add_to)
