"""Which requests run in the next step, and with how many tokens.

The rules are the reference's (nanovllm/engine/scheduler.py:380-983): running
requests decode first (policy ``decode_first``) or wait while prompts are pending
(``prefill_first``); what is left of the token budget goes to waiting prompts in
arrival order, the head of the queue only, cut to the budget, so at most one
unfinished portion is in a step; a prompt that has waited longer than
``max_prefill_wait_ms`` gets one request's place and one token reserved and may
push running requests out. When a decoding request needs a page and none is free,
the running request with the fewest cached tokens is pushed out and computed again
later (prompt and generated tokens), or, if there is no other, the request itself.

Unlike the reference, whose step runs a decode pass and then a prefill pass, the
plan here is one batch: decoding requests first, then prompt portions.
"""
from __future__ import annotations

from collections import deque
from dataclasses import dataclass, field
from time import monotonic
from typing import Callable

from ..cache.manager import CacheManager
from .sequence import Sequence, SequenceStatus


@dataclass
class SchedulePlan:
    """One step: ``seqs[i]`` feeds its next ``seqs[i].num_scheduled_tokens`` tokens."""

    decode_seqs: list[Sequence] = field(default_factory=list)
    prefill_seqs: list[Sequence] = field(default_factory=list)
    preempted_seq_ids: list[int] = field(default_factory=list)

    @property
    def seqs(self) -> list[Sequence]:
        return self.decode_seqs + self.prefill_seqs

    @property
    def num_decode_tokens(self) -> int:
        return len(self.decode_seqs)

    @property
    def num_prefill_tokens(self) -> int:
        return sum(s.num_scheduled_tokens for s in self.prefill_seqs)

    @property
    def is_empty(self) -> bool:
        return not self.decode_seqs and not self.prefill_seqs


class Scheduler:
    def __init__(self, cache: CacheManager, max_num_seqs: int, max_num_batched_tokens: int, eos: int,
                 max_model_len: int, scheduler_policy: str = "decode_first", max_prefill_wait_ms: float = 50.0,
                 clock: Callable[[], float] = monotonic):
        if scheduler_policy not in ("decode_first", "prefill_first"):
            raise ValueError("scheduler_policy must be 'decode_first' or 'prefill_first'")
        self.cache = cache
        self.max_num_seqs = max_num_seqs
        self.max_num_batched_tokens = max_num_batched_tokens
        self.max_model_len = max_model_len
        self.eos = eos
        self.scheduler_policy = scheduler_policy
        self.max_prefill_wait_ms = max_prefill_wait_ms
        self.clock = clock
        self.waiting: deque[Sequence] = deque()
        self.running: deque[Sequence] = deque()
        self.waiting_since: dict[int, float] = {}
        self.num_preemptions = 0
        self.num_recomputed_tokens = 0

    # ------------------------------------------------------------------ intake
    def add(self, seq: Sequence) -> None:
        """Refuses at once what could never run: a request longer than the model
        allows or than all pages together (the reference finds out only when the
        scheduler stops making progress, scheduler.py:898-903)."""
        longest = seq.num_prompt_tokens + seq.max_tokens
        if longest > self.max_model_len:
            raise ValueError(f"prompt of {seq.num_prompt_tokens} tokens and max_tokens {seq.max_tokens} "
                             f"exceed max_model_len {self.max_model_len}")
        for g in self.cache.groups:
            if -(-longest // g.page_size) > g.num_pages:
                raise ValueError(f"a request of up to {longest} tokens needs {-(-longest // g.page_size)} pages; "
                                 f"the cache has {g.num_pages}")
        self.waiting.append(seq)
        self.waiting_since[seq.seq_id] = self.clock()

    def is_finished(self) -> bool:
        return not self.waiting and not self.running

    # ------------------------------------------------------------------ helpers
    def _head_waited_too_long(self, now: float) -> bool:
        if not self.waiting:
            return False
        since = self.waiting_since.get(self.waiting[0].seq_id, now)
        return (now - since) * 1000.0 >= self.max_prefill_wait_ms

    def _select_preemption_victim(self, excluded: set[int] = frozenset()) -> Sequence | None:
        """The running request that costs least to compute again (scheduler.py:350-378)."""
        candidates = [s for s in self.running if s.seq_id not in excluded]
        if not candidates:
            return None
        return min(candidates, key=lambda s: (s.num_cached_tokens, s.seq_id))

    def preempt(self, seq: Sequence) -> None:
        """Gives back all the request holds and queues it again at the tail; the caller
        has taken it out of ``running`` (scheduler.py:906-949)."""
        self.num_preemptions += 1
        self.num_recomputed_tokens += seq.num_cached_tokens
        seq.status = SequenceStatus.WAITING
        seq.num_cached_tokens = 0
        seq.num_scheduled_tokens = 0
        if seq.seq_id in self.cache:
            self.cache.release(seq.seq_id)
        self.waiting.append(seq)
        self.waiting_since[seq.seq_id] = self.clock()

    # ------------------------------------------------------------------ the plan
    def schedule(self) -> SchedulePlan:
        plan = SchedulePlan()
        now = self.clock()
        strict_prefill_first = self.scheduler_policy == "prefill_first" and bool(self.waiting)
        reserve_prefill = strict_prefill_first or self._head_waited_too_long(now)
        if strict_prefill_first:
            decode_seq_limit = decode_token_limit = 0
        else:
            decode_seq_limit = max(0, self.max_num_seqs - (1 if reserve_prefill else 0))
            decode_token_limit = max(0, self.max_num_batched_tokens - (1 if reserve_prefill else 0))

        # 1. every running request decodes one token
        while self.running and len(plan.decode_seqs) < decode_seq_limit and len(plan.decode_seqs) < decode_token_limit:
            seq = self.running.popleft()
            # its last token goes into the cache in this step: position len - 1
            while not self.cache.can_reserve(seq.seq_id, seq.num_tokens):
                victim = self._select_preemption_victim()
                if victim is None:
                    plan.preempted_seq_ids.append(seq.seq_id)
                    self.preempt(seq)
                    seq = None
                    break
                plan.preempted_seq_ids.append(victim.seq_id)
                self.running.remove(victim)
                self.preempt(victim)
            if seq is None:
                continue
            self.cache.reserve(seq.seq_id, seq.num_tokens)
            seq.num_scheduled_tokens = seq.num_tokens - seq.num_cached_tokens      # always 1
            plan.decode_seqs.append(seq)
        self.running.extendleft(reversed(plan.decode_seqs))
        scheduled_decode_ids = {s.seq_id for s in plan.decode_seqs}

        # 2. what is left goes to the head of the waiting queue
        remaining_tokens = self.max_num_batched_tokens - len(plan.decode_seqs)
        remaining_seqs = self.max_num_seqs - len(plan.decode_seqs)
        num_active = len(self.running) + sum(1 for s in self.waiting if s.seq_id in self.cache)
        while self.waiting and len(plan.prefill_seqs) < remaining_seqs and remaining_tokens > 0:
            seq = self.waiting[0]
            if seq.seq_id not in self.cache:
                def resources_available() -> bool:
                    return num_active < self.max_num_seqs and self.cache.can_start(seq.token_ids)
                while reserve_prefill and not resources_available():
                    # requests that already have a place in this step stay: the decoding ones and (unlike
                    # the reference, scheduler.py:674-719, which would push them out) the prompts just planned
                    victim = self._select_preemption_victim(
                        scheduled_decode_ids | {p.seq_id for p in plan.prefill_seqs})
                    if victim is None:
                        break
                    plan.preempted_seq_ids.append(victim.seq_id)
                    self.running.remove(victim)
                    self.preempt(victim)
                    num_active -= 1
                if not resources_available():
                    break
                # pages for the whole request as it stands (prompt, and generated tokens of a request
                # that is computed again), so that no portion can run out of pages (block_manager.py:696-749)
                self.cache.admit(seq.seq_id, seq.token_ids)
                self.cache.reserve(seq.seq_id, seq.num_tokens)
                # with shared prefixes the first pages may hold this request's first tokens already
                # (nanovllm/engine/block_manager.py:727-749)
                seq.num_cached_tokens = self.cache.num_tokens(seq.seq_id)
                num_active += 1
            left = seq.num_tokens - seq.num_cached_tokens
            if left <= 0:
                raise RuntimeError(f"request {seq.seq_id} waits but has no tokens left to feed")
            seq.num_scheduled_tokens = min(left, remaining_tokens)
            remaining_tokens -= seq.num_scheduled_tokens
            plan.prefill_seqs.append(seq)
            if seq.num_cached_tokens + seq.num_scheduled_tokens == seq.num_tokens:
                seq.status = SequenceStatus.RUNNING
                self.waiting.popleft()
                self.waiting_since.pop(seq.seq_id, None)
                self.running.append(seq)
            else:
                self.waiting_since[seq.seq_id] = self.clock()       # its wait starts again
        if plan.is_empty:
            raise RuntimeError("Scheduler cannot make progress: no decode or prefill request could be scheduled")
        return plan

    # ------------------------------------------------------------------ after the step
    def postprocess(self, seqs: list[Sequence], token_ids: list[int | None]) -> list[Sequence]:
        """``token_ids[i]`` is the token sampled for ``seqs[i]`` (None for a portion that
        does not end its request's tokens). Returns the requests that finished
        (scheduler.py:972-983)."""
        finished = []
        for seq, token_id in zip(seqs, token_ids):
            seq.num_cached_tokens += seq.num_scheduled_tokens
            seq.num_scheduled_tokens = 0
            if seq.num_cached_tokens < seq.num_tokens:
                continue
            if token_id is None:
                raise RuntimeError(f"request {seq.seq_id} fed its last token but got no sampled token")
            seq.append_token(token_id)
            if (not seq.ignore_eos and token_id == self.eos) or seq.num_completion_tokens == seq.max_tokens:
                seq.status = SequenceStatus.FINISHED
                self.cache.release(seq.seq_id)
                self.running.remove(seq)
                finished.append(seq)
        return finished
