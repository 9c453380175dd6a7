"""How a layer's norm, mixer and feed-forward are arranged."""
from __future__ import annotations

from .base import BLOCKS, Part


@BLOCKS.register("prenorm")
class PreNormBlock(Part):
    """r += mixer(norm(r)); r += feed_forward(norm(r)), with each addition folded into
    the next norm (nanovllm/models/qwen3.py:152-159): the block takes and returns
    (hidden, residual), and ``residual`` is None before the first block."""

    # the norms this arrangement takes, by the names of its constructor's arguments: the model builds one per slot
    # from the layer's description (``LayerSpec.norms[slot]``, else ``LayerSpec.norm``)
    norm_slots = ("mixer_norm", "feed_forward_norm")

    def __init__(self, mixer, feed_forward, mixer_norm, feed_forward_norm):
        self.mixer = mixer
        self.feed_forward = feed_forward
        self.mixer_norm = mixer_norm
        self.feed_forward_norm = feed_forward_norm

    def children(self):
        return {"mixer_norm": self.mixer_norm, "mixer": self.mixer,
                "feed_forward_norm": self.feed_forward_norm, "feed_forward": self.feed_forward}

    def forward(self, hidden, residual, step, cache):
        if residual is None:
            x, residual = self.mixer_norm.forward_start(hidden)
        else:
            x, residual = self.mixer_norm.forward_add(hidden, residual)
        x = self.mixer.forward(x, step, cache)
        x, residual = self.feed_forward_norm.forward_add(x, residual)
        x = self.feed_forward.forward(x, step)
        return x, residual
