"""Per-request sampling options: the reference's three fields
(nanovllm/sampling_params.py:5-15) and a seed."""
from __future__ import annotations

import math
from dataclasses import dataclass


@dataclass
class SamplingParams:
    temperature: float = 1.0      # 0: greedy
    max_tokens: int = 64
    ignore_eos: bool = False
    seed: int | None = None       # None: the engine's seed

    def __post_init__(self):
        if not math.isfinite(self.temperature):
            raise ValueError("temperature must be finite")
        if self.temperature < 0:
            raise ValueError("temperature must be non-negative")
        if isinstance(self.max_tokens, bool) or not isinstance(self.max_tokens, int) or self.max_tokens <= 0:
            raise ValueError("max_tokens must be a positive integer")
