"""Trace replay: given token ids go through the step function, step by step, and the
logits of the wanted places come back. Nothing is sampled and nothing is scheduled:
the trace says which request brings which tokens in which step.

A step is a dict, one line of JSON in a trace file:

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": ["b"]}

``entries``: for each request its next tokens and the places among them whose logits
are wanted; all entries of a step are one batch. ``end``: requests that are over
after this step; what they hold in the cache is given back. An entry may also bring
``"positions": [[...], ...]``, its tokens' positions as the position encodings see
them, one list per position axis of the model (default: the tokens' indices).

A whole trace may also come as one JSON object that names the requests' tokens once and
then says, step by step, how many of its next tokens each request feeds:

    {"requests": {"a": [5, 17, 3, 9], "b": [1, 2]}, "steps": [[{"req": "a", "n": 3}], [{"req": "a", "n": 1}, {"req": "b", "n": 2}]],
     "dtype": "float32", "block_size": 64, "num_blocks": 8, "model": "DIR"}        (or "shape": "tinyB", "seed": 1)

``steps_of_trace`` turns it into steps of the first kind: the logits of every fed position are
wanted, and a request ends with its last token. ``bin/trace_run --trace FILE --out X.safetensors``
then writes ``{request: [its length, vocab]}``.

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
    entries = [StepEntry(e["id"], list(e["tokens"]), list(e.get("want") or []), e.get("positions"))
               for e in record.get("entries") or []]
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


def steps_of_trace(trace: dict) -> list[dict]:
    """The steps of a trace that is one object (see the module's text), as the records that ``replay_step`` takes.
    Everything that is wrong with the trace is an error here, before any step has run."""
    requests = trace.get("requests")
    if not isinstance(requests, dict) or not requests or not isinstance(trace.get("steps"), list):
        raise ValueError("a trace holds 'requests': {id: [token ids]} and 'steps': [[{'req': id, 'n': count}, ...], ...]")
    fed = {rid: 0 for rid in requests}
    records = []
    for number, step in enumerate(trace["steps"]):
        entries, ended = [], []
        for item in step:
            rid, n = item.get("req"), item.get("n")
            if rid not in requests:
                raise ValueError(f"step {number}: request {rid!r} is not among the trace's requests")
            if not isinstance(n, int) or n <= 0 or fed[rid] + n > len(requests[rid]):
                raise ValueError(f"step {number}: request {rid!r} cannot feed {n!r} tokens after {fed[rid]} of its "
                                 f"{len(requests[rid])}")
            entries.append({"id": rid, "tokens": list(requests[rid][fed[rid]:fed[rid] + n]), "want": list(range(n))})
            fed[rid] += n
            if fed[rid] == len(requests[rid]):
                ended.append(rid)
        records.append({"step": number, "entries": entries, "end": ended})
    unfinished = sorted(str(rid) for rid, n in fed.items() if n != len(requests[rid]))
    if unfinished:
        raise ValueError(f"the steps do not feed all tokens of request(s) {', '.join(unfinished)}")
    return records


def peak_tokens_of(records: list[dict], unit: int = 64) -> int:
    """The most tokens that live requests hold at any time in these steps, each request's count rounded up to a
    multiple of ``unit``: what ``make_runner`` sizes the cache for."""
    held: dict = {}
    peak = 0
    for record in records:
        for e in record.get("entries") or []:
            held[e["id"]] = held.get(e["id"], 0) + len(e["tokens"])
        peak = max(peak, sum(-(-n // unit) * unit for n in held.values()))
        for rid in record.get("end") or []:
            held.pop(rid, None)
    return peak
