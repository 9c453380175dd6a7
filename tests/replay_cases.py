"""Traces for the replay tests: the same requests cut into steps in different ways.

A trace is a list of steps in the format of ``bin/trace_run``:
``{"step": n, "entries": [{"id", "tokens", "want"}], "end": [ids]}``.
Every trace here wants the logits of every token it feeds, so that any two ways of
cutting the same requests can be compared position by position with each other
and with the plain whole-sequence implementation.
"""
from __future__ import annotations

import torch


def random_tokens(vocab: int, n: int, seed: int) -> list[int]:
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def _entry(rid, tokens):
    return {"id": rid, "tokens": list(tokens), "want": list(range(len(tokens)))}


def whole(requests: dict[str, list[int]]) -> list[dict]:
    """Each request alone and whole, one after the other."""
    return [{"step": i, "entries": [_entry(rid, toks)], "end": [rid]}
            for i, (rid, toks) in enumerate(requests.items())]


def tail_decoded(requests: dict[str, list[int]], tail: int = 32) -> list[dict]:
    """Most of a request in one step, then its last ``tail`` tokens one by one."""
    steps = []
    for rid, toks in requests.items():
        head = max(1, len(toks) - tail)
        steps.append({"step": len(steps), "entries": [_entry(rid, toks[:head])], "end": []})
        for i in range(head, len(toks)):
            steps.append({"step": len(steps), "entries": [_entry(rid, toks[i:i + 1])],
                          "end": [rid] if i == len(toks) - 1 else []})
        if head == len(toks):
            steps[-1]["end"] = [rid]
    return steps


def portions(requests: dict[str, list[int]], sizes=(7, 2, 5, 3, 2, 11, 1, 4, 2, 9)) -> list[dict]:
    """Portions of changing size, down to two tokens (and one)."""
    steps = []
    for rid, toks in requests.items():
        i, k = 0, 0
        while i < len(toks):
            n = min(sizes[k % len(sizes)], len(toks) - i)
            k += 1
            steps.append({"step": len(steps), "entries": [_entry(rid, toks[i:i + n])],
                          "end": [rid] if i + n == len(toks) else []})
            i += n
    return steps


def mixed(requests: dict[str, list[int]], max_live: int = 4, prompt_fraction: float = 0.6,
          sizes=(5, 2, 9, 3, 16, 2, 7), skip_every: int = 5) -> list[dict]:
    """Up to ``max_live`` requests at a time. Each request is fed the first part of its
    tokens in portions and the rest one token a step; a step holds portions of some
    requests beside single tokens of others; every ``skip_every``-th step one live
    request is left out. A request that ends frees its pages for the next one."""
    waiting = list(requests.items())
    live: dict[str, dict] = {}
    steps = []
    k = 0
    while waiting or live:
        while waiting and len(live) < max_live:
            rid, toks = waiting.pop(0)
            live[rid] = {"tokens": toks, "fed": 0, "prompt": max(1, int(len(toks) * prompt_fraction))}
        entries, end = [], []
        ids = list(live)
        skipped = ids[len(steps) % len(ids)] if (len(steps) % skip_every == skip_every - 1 and len(ids) > 1) else None
        for rid in ids:
            if rid == skipped:
                continue
            st = live[rid]
            if st["fed"] < st["prompt"]:
                n = min(sizes[k % len(sizes)], st["prompt"] - st["fed"])
                k += 1
            else:
                n = 1
            entries.append(_entry(rid, st["tokens"][st["fed"]:st["fed"] + n]))
            st["fed"] += n
            if st["fed"] == len(st["tokens"]):
                end.append(rid)
        for rid in end:
            del live[rid]
        steps.append({"step": len(steps), "entries": entries, "end": end})
    return steps


def peak_tokens(steps: list[dict], page: int = 64) -> int:
    """The most tokens that live requests hold at any time, each rounded up to a page."""
    held: dict[str, int] = {}
    peak = 0
    for st in steps:
        for e in st["entries"]:
            held[e["id"]] = held.get(e["id"], 0) + len(e["tokens"])
        peak = max(peak, sum(-(-n // page) * page for n in held.values()))
        for rid in st["end"]:
            held.pop(rid, None)
    return peak


def run_in_process(runner, steps: list[dict]) -> dict[str, torch.Tensor]:
    """A trace through the replay program's own function, in this process: per request the logits of all its
    tokens, in order."""
    from nanohybrid_vlm_amd.engine.replay import replay

    return replay(runner, steps)
