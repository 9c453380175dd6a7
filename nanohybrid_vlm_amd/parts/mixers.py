"""Token mixers. ``GQAAttention`` follows nanovllm/models/qwen3.py:14-88 and
nanovllm/layers/attention.py:43-75."""
from __future__ import annotations

import torch

from ..native import ops
from .base import MIXERS, CacheView, PagedKVNeed, ParamSpec, Part


@MIXERS.register("gqa_attention")
class GQAAttention(Part):
    """Causal attention with grouped key/value heads over the paged cache.

    qkv = x W^T (+ b), rows of W ordered q | k | v (nanovllm/layers/linear.py:150-167);
    optional RMSNorm over each q and k head (qwen3.py:82-84); rotation; keys (normed
    and turned) and values are stored at the step's slots; every query reads its
    request's keys up to its own position (attention.py:64-74); output projection
    without bias (qwen3.py:49-53).
    """

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int, scale: float,
                 qk_norm_eps: float | None, qkv_bias: bool, position, window: int | None = None):
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} heads are not a multiple of {num_kv_heads} key/value heads")
        self.hidden_size = hidden_size
        self.num_heads = num_heads
        self.num_kv_heads = num_kv_heads
        self.head_dim = head_dim
        self.scale = scale
        self.qk_norm_eps = qk_norm_eps
        self.qkv_bias = qkv_bias
        self.position = position
        self.window = window
        self.qkv_weight = self.qkv_bias_t = self.o_weight = None
        self.q_norm_weight = self.k_norm_weight = None

    def param_specs(self):
        width = (self.num_heads + 2 * self.num_kv_heads) * self.head_dim
        specs = {
            "qkv.weight": ParamSpec((width, self.hidden_size)),
            "o.weight": ParamSpec((self.hidden_size, self.num_heads * self.head_dim)),
        }
        if self.qkv_bias:
            specs["qkv.bias"] = ParamSpec((width,), init="zeros")
        if self.qk_norm_eps is not None:
            specs["q_norm.weight"] = ParamSpec((self.head_dim,), init="norm", keeps_float32=True)
            specs["k_norm.weight"] = ParamSpec((self.head_dim,), init="norm", keeps_float32=True)
        return specs

    def bind(self, params):
        self.qkv_weight = params["qkv.weight"]
        self.o_weight = params["o.weight"]
        self.qkv_bias_t = params.get("qkv.bias")
        self.q_norm_weight = params.get("q_norm.weight")
        self.k_norm_weight = params.get("k_norm.weight")

    def cache_need(self):
        return PagedKVNeed(self.num_kv_heads, self.head_dim, self.window)

    takes_deferred_norm = True    # x goes straight into a product, which can norm it
    adds_to_residual = True       # the output projection can make the addition to the residual stream

    def first_product(self):
        """(weight, gated) of the product that x goes into."""
        return self.qkv_weight, False

    def forward(self, x, step, cache: CacheView, add_to=None):
        tables = step.groups[cache.group]
        qkv = ops.linear(x, self.qkv_weight)
        # an encoding over several position axes says which axis turns each pair; others turn by the first axis
        pair_axes = self.position.pair_axes() if hasattr(self.position, "pair_axes") else None
        q = ops.qk_rope_write(
            qkv, self.qkv_bias_t, self.q_norm_weight, self.k_norm_weight,
            self.qk_norm_eps if self.qk_norm_eps is not None else 0.0,
            self.position.rotation_table(), step.token_positions if pair_axes is None else step.positions,
            tables.slot_mapping, cache.k, cache.v, self.num_heads, self.num_kv_heads, self.head_dim,
            write_kv=cache.writes, pair_axes=pair_axes)
        o = ops.paged_attention(q, cache.k, cache.v, step.attention, tables.block_tables, self.scale, self.window)
        return ops.linear(o.view(o.shape[0], self.num_heads * self.head_dim), self.o_weight, add_to=add_to)
