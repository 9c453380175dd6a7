"""What a request asks of sampling: the reference's three fields
(nanovllm/sampling_params.py:5-15: temperature, max_tokens, ignore_eos) and a seed."""
from __future__ import annotations

from dataclasses import dataclass


@dataclass
class SamplingParams:
    temperature: float = 1.0      # 0: the most likely token is taken
    max_tokens: int = 64          # tokens to generate at most
    ignore_eos: bool = False      # True: the end-of-sequence token does not end the request
    seed: int | None = None       # None: the engine's seed

    def __post_init__(self):
        t = self.temperature
        if isinstance(t, bool) or not isinstance(t, (int, float)):
            raise TypeError(f"temperature is a number, got {t!r}")
        # a NaN fails both comparisons, an infinity the second
        if not (0.0 <= t < float("inf")):
            raise ValueError(f"temperature {t!r}: a finite number that is 0 (greedy) or above is needed")
        n = self.max_tokens
        if isinstance(n, bool) or not isinstance(n, int) or n < 1:
            raise ValueError(f"max_tokens {n!r}: a whole number of at least 1 is needed")
        if self.seed is not None and (isinstance(self.seed, bool) or not isinstance(self.seed, int)):
            raise TypeError(f"seed is an integer or None, got {self.seed!r}")
