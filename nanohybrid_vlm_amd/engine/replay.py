"""Trace replay: given token ids go through the step function, step by step, and the
logits of the wanted places come back. Nothing is sampled and nothing is scheduled:
the trace says which request brings which tokens in which step.

A step is a dict, one line of JSON in a trace file:

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": ["b"]}

``entries``: for each request its next tokens and the places among them whose logits
are wanted; all entries of a step are one batch. ``end``: requests that are over
after this step; what they hold in the cache is given back.

``bin/trace_run`` and the tests' in-process replays both go through ``replay_step``,
so the program and the tests drive the engine in the same way. The reference has
nothing like it; the nearest is stepping its engine by hand
(tests/5090-test-TP2/run_generation.py:62-134).
"""
from __future__ import annotations

import math

import torch

from .runner import ModelRunner, StepEntry


def pages_for(max_tokens: int, page_size: int, max_live: int = 4, unit: int = 64) -> int:
    """Pages that hold ``max_tokens`` tokens of up to ``max_live`` requests, when the caller counted every
    request's tokens rounded up to a multiple of ``unit``. A page size that divides ``unit`` needs exactly
    ``max_tokens / page_size``; any other loses up to ``page_size - gcd(page_size, unit)`` more tokens a request
    to its last page."""
    if max_tokens <= 0 or page_size <= 0:
        raise ValueError("max_tokens and page_size must be positive")
    if unit % page_size == 0:
        return -(-max_tokens // page_size)
    return -(-(max_tokens + max_live * (page_size - math.gcd(page_size, unit))) // page_size)


def make_runner(model_dir: str, dtype: str, max_tokens: int, page_size: int = 64, device: str = "cuda:0",
                use_graphs: bool = True, max_live: int = 4, **runner_options) -> ModelRunner:
    """The runner of a replay: a cache pool made for ``max_tokens`` and no more, so that pages are used again."""
    num_pages = pages_for(max_tokens, page_size, max_live)
    return ModelRunner(model_dir, dtype=dtype, device=device, page_size=page_size, num_pages=num_pages,
                       num_state_slots=max(max_live, 1), use_graphs=use_graphs, max_model_len=num_pages * page_size,
                       **runner_options)


def replay_step(runner: ModelRunner, record: dict) -> torch.Tensor | None:
    """Runs one step of a trace. Returns float32 logits [wanted, vocab] in the order of the entries and of each
    entry's ``want``, or None if the step wants nothing (or brings nothing)."""
    entries = [StepEntry(e["id"], list(e["tokens"]), list(e.get("want") or [])) for e in record.get("entries") or []]
    logits = runner.step(entries) if entries else None
    for request_id in record.get("end") or []:
        runner.finish(request_id)
    return logits


def replay(runner: ModelRunner, steps) -> dict:
    """Runs a whole trace; returns for every request the logits of all its wanted places, in the order in which
    they were fed: {id: [places, vocab]} on the CPU. The cache manager's invariants are checked after every step."""
    parts: dict = {}
    for record in steps:
        logits = replay_step(runner, record)
        row = 0
        for e in record.get("entries") or []:
            n = len(e.get("want") or [])
            if n:
                parts.setdefault(e["id"], []).append(logits[row:row + n].float().cpu())
                row += n
        runner.cache.check()
    return {rid: torch.cat(p) for rid, p in parts.items()}
