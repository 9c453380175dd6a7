"""Greedy and temperature sampling of one token per row of logits.

The reference (nanovllm/layers/sampler.py:6-65) takes the argmax for rows with
temperature 0 and, for the others, argmax(softmax(logits / T) / e) with e ~ Exp(1)
drawn from torch's global generator. The same is done here in one HIP kernel, with
the noise a function of (seed, request, number of the token, vocabulary index)
only: what a request samples does not depend on what else is in the batch or on
how its prompt was cut. A batch of greedy rows uses no randomness at all.
"""
from __future__ import annotations

import torch

from ..native import ops

_MASK = (1 << 64) - 1


def _mix(z: int) -> int:
    z = (z + 0x9E3779B97F4A7C15) & _MASK
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _MASK
    return z ^ (z >> 31)


def noise_key(seed: int, request: int, step: int) -> int:
    """The 64-bit key of one draw, as a signed integer (for an int64 tensor)."""
    key = _mix(_mix(_mix(seed & _MASK) ^ (request & _MASK)) ^ (step & _MASK))
    return key - (1 << 64) if key >= (1 << 63) else key


class Sampler:
    def __init__(self, vocab_size: int):
        self.vocab_size = vocab_size

    def __call__(self, logits: torch.Tensor, temperatures: list[float], keys: list[int]) -> list[int]:
        """``logits``: float32 [n, vocab] on the device; one temperature and one key per row."""
        n = logits.shape[0]
        if len(temperatures) != n or len(keys) != n:
            raise ValueError(f"{n} rows of logits, {len(temperatures)} temperatures, {len(keys)} keys")
        temps = torch.tensor(temperatures, dtype=torch.float32).to(logits.device, non_blocking=True)
        keys_t = torch.tensor(keys, dtype=torch.int64).to(logits.device, non_blocking=True)
        tokens = ops.sample(logits, temps, keys_t).tolist()
        for t in tokens:
            if not 0 <= t < self.vocab_size:
                raise RuntimeError("sampling met logits that are not numbers")
        return tokens
