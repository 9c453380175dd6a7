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
        self._staged = None          # on a GPU: pinned host memory and its device twin for temperatures, keys and tokens

    def _stage(self, n: int, device) -> dict:
        """Pinned host buffers and their device twins for ``n`` rows. What a step passes to the kernel and gets
        back goes through them with copies that do not block: a copy from ordinary host memory makes the host
        wait until the GPU has caught up, twice a step, before the kernel is even launched."""
        st = self._staged
        if st is None or st["rows"] < n or st["device"] != device:
            rows = max(64, 2 * n)
            st = self._staged = {
                "rows": rows, "device": device,
                "host_temps": torch.empty(rows, dtype=torch.float32, pin_memory=True),
                "host_keys": torch.empty(rows, dtype=torch.int64, pin_memory=True),
                "host_tokens": torch.empty(rows, dtype=torch.int32, pin_memory=True),
                "temps": torch.empty(rows, dtype=torch.float32, device=device),
                "keys": torch.empty(rows, dtype=torch.int64, device=device),
                "done": torch.cuda.Event(),
            }
        return st

    def __call__(self, logits: torch.Tensor, temperatures: list[float], keys: list[int]) -> list[int]:
        """``logits``: float32 [n, vocab] on the device; one temperature and one key per row."""
        return self.finish(self.launch(logits, temperatures, keys))

    def launch(self, logits: torch.Tensor, temperatures: list[float], keys: list[int]) -> dict:
        """Asks for the tokens without waiting for them; ``finish`` waits. ``["tokens"]`` of the result is the
        int32 tensor on the device that will hold them (a caller may feed it to the next step meanwhile)."""
        n = logits.shape[0]
        if len(temperatures) != n or len(keys) != n:
            raise ValueError(f"{n} rows of logits, {len(temperatures)} temperatures, {len(keys)} keys")
        if logits.device.type != "cuda":
            temps = torch.tensor(temperatures, dtype=torch.float32).to(logits.device)
            keys_t = torch.tensor(keys, dtype=torch.int64).to(logits.device)
            return {"n": n, "tokens": ops.sample(logits, temps, keys_t), "staged": None}
        st = self._stage(n, logits.device)
        st["host_temps"][:n] = torch.tensor(temperatures, dtype=torch.float32)
        st["host_keys"][:n] = torch.tensor(keys, dtype=torch.int64)
        st["temps"][:n].copy_(st["host_temps"][:n], non_blocking=True)
        st["keys"][:n].copy_(st["host_keys"][:n], non_blocking=True)
        tokens = ops.sample(logits, st["temps"][:n], st["keys"][:n])
        st["host_tokens"][:n].copy_(tokens, non_blocking=True)
        st["done"].record()
        return {"n": n, "tokens": tokens, "staged": st}

    def finish(self, launched: dict) -> list[int]:
        st, n = launched["staged"], launched["n"]
        if st is None:
            tokens = launched["tokens"].tolist()
        else:
            st["done"].synchronize()
            tokens = st["host_tokens"][:n].tolist()
        for t in tokens:
            if not 0 <= t < self.vocab_size:
                raise RuntimeError("sampling met logits that are not numbers")
        return tokens
