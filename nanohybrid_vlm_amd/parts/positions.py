"""Position encodings. A position encoding hands the mixer a table of rotation
angles (cosines and sines per position) or nothing; the mixer's kernel turns
queries and keys by it before they are used and stored. A token's position may
have several coordinates (``ModelSpec.position_axes``; a step carries them as
[axes, tokens]): an encoding over several axes also says, pair by pair, which
axis' coordinate looks up the pair's angle (``pair_axes``)."""
from __future__ import annotations

import torch

from .base import POSITION_ENCODINGS, Part


class PositionEncoding(Part):
    """What a mixer asks of its position encoding."""

    def rotation_table(self) -> torch.Tensor | None:
        """[max_position, rotary_dim] float32 (cosines | sines), or None: nothing is turned."""
        return None

    def pair_axes(self) -> torch.Tensor | None:
        """[rotary_dim / 2] int32: the position axis that turns each pair; None: all turn by the first axis."""
        return None

    def to(self, device):
        return self


@POSITION_ENCODINGS.register("rope")
class RotaryEmbedding(PositionEncoding):
    """nanovllm/layers/rotary_embedding.py:83-89: inv_freq_j = base^(-2j/rotary_dim),
    table[p] = [cos(p * inv_freq) | sin(p * inv_freq)] in float32. The rotation
    itself (first half against second half, rotary_embedding.py:6-14) is done by
    the mixer's kernel."""

    def __init__(self, rotary_dim: int, max_position: int, base: float, device=None):
        if rotary_dim % 2:
            raise ValueError(f"rotary_dim must be even, got {rotary_dim}")
        self.rotary_dim = rotary_dim
        self.max_position = max_position
        self.base = base
        inv_freq = 1.0 / (base ** (torch.arange(0, rotary_dim, 2, dtype=torch.float32) / rotary_dim))
        t = torch.arange(max_position, dtype=torch.float32)
        freqs = torch.einsum("i,j->ij", t, inv_freq)
        self.table = torch.cat((freqs.cos(), freqs.sin()), dim=-1).contiguous()   # [max_position, rotary_dim]
        if device is not None:
            self.table = self.table.to(device)

    def rotation_table(self) -> torch.Tensor | None:
        return self.table

    def to(self, device):
        self.table = self.table.to(device)
        return self


@POSITION_ENCODINGS.register("none")
class NoPositions(PositionEncoding):
    """No position signal at all (attention then depends on order only through the mask)."""

    def __init__(self, max_position: int, device=None):
        self.max_position = max_position

    def rotation_table(self):
        return None

    def to(self, device):
        return self
