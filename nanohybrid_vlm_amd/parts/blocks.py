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

    @property
    def takes_summed(self) -> bool:
        """Whether ``hidden`` may come as an ``ops.Summed`` (the block before has added it to the residual stream
        already): this block's first norm has to know what that is. A block that says so takes ``next_norm=``."""
        return getattr(self.mixer_norm, "takes_summed", False)

    def forward(self, hidden, residual, step, cache, next_norm=None, next_reader=None):
        """``next_norm``: the norm that takes this block's result next (the next block's first norm, or the model's
        last), if it takes an ``ops.Summed`` in place of ``hidden``; ``next_reader``: the part that reads that norm."""
        # A mixer or feed-forward that says ``adds_to_residual`` takes ``add_to=`` (the residual stream and the norm
        # that follows, ``ops.AddTo``) and may let its last product make the addition (it then returns an
        # ``ops.Summed``); one that says ``takes_deferred_norm`` may get an ``ops.Normed`` as its input, whose rows
        # its first product scales. Parts that say neither get tensors and return tensors.
        mixer, ff = self.mixer, self.feed_forward
        if residual is None:
            x, residual = self.mixer_norm.forward_start(hidden)
        else:
            x, residual = self.mixer_norm.forward_add(hidden, residual, **_deferred(self.mixer_norm, mixer))
        x = mixer.forward(x, step, cache, **_add_to(mixer, self.feed_forward_norm, residual, ff))
        x, residual = self.feed_forward_norm.forward_add(x, residual, **_deferred(self.feed_forward_norm, ff))
        x = ff.forward(x, step, **_add_to(ff, next_norm, residual, next_reader))
        return x, residual


def _deferred(norm, reader) -> dict:
    """The argument that lets ``norm`` hand its scaling on to ``reader``, if both are made for that."""
    both = getattr(norm, "defers_to_products", False) and getattr(reader, "takes_deferred_norm", False)
    return {"deferred": True} if both else {}


def _add_to(part, norm, residual, reader) -> dict:
    """The argument that lets ``part`` make the addition that ``norm`` would make, if both are made for that.
    ``reader``: the part that reads ``norm`` (it counts only if it takes the norm with its scaling left to do)."""
    if norm is not None and getattr(part, "adds_to_residual", False) and getattr(norm, "takes_summed", False):
        return {"add_to": norm.add_to(residual, reader if getattr(reader, "takes_deferred_norm", False) else None)}
    return {}
