"""Which requests run in the next step, and with how many tokens.

A step here is one batch, so a plan is one list: the requests that decode (one
token each) followed by the prompts that are fed (a portion each). The plan is
made in two passes over the two queues, each a method of its own:

* ``_decoding_pass`` walks ``running`` in its order and gives every request its
  next token, taking a page for it where the token starts one. When no page is
  free, a request is pushed out (see ``_push_out``) until one is.
* ``_admission_pass`` spends what the step has left on the head of ``waiting``:
  admits it if it is new (state slot and pages for all it holds, so no later
  portion can run out of pages), and feeds it as many tokens as are left. A
  prompt that is not finished stays at the head; only the head is ever looked at,
  so requests start in arrival order and a step holds at most one unfinished
  portion.

The rules themselves are the reference's (nanovllm/engine/scheduler.py:380-983):
the two policies (``decode_first``: decoding always goes on and prompts get the
rest of the token budget; ``prefill_first``: nothing decodes while a prompt
waits), first-come admission of the head only, recomputation as the answer to a
cache that is full (the request with the fewest stored tokens goes, ties to the
older one, and comes back at the tail with prompt and generated tokens as its new
prompt), a prompt that has waited ``max_prefill_wait_ms`` gets a place and a token
kept free in the decoding pass and may push running requests out. The reference
runs a decode pass and a prefill pass of the model per step; its two budgets are
shared by both, as they are here by the one batch.
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


@dataclass
class _Room:
    """What a step can still take: tokens of the batch and requests in it."""

    tokens: int
    requests: int

    def take(self, tokens: int) -> None:
        self.tokens -= tokens
        self.requests -= 1

    @property
    def left(self) -> bool:
        return self.tokens > 0 and self.requests > 0


class Scheduler:
    def __init__(self, cache: CacheManager, max_num_seqs: int, max_num_batched_tokens: int, eos: int,
                 max_model_len: int, scheduler_policy: str = "decode_first", max_prefill_wait_ms: float = 50.0,
                 clock: Callable[[], float] = monotonic, release: Callable | None = None):
        """``release``: how a request's pages and state slot are given back (default: the cache manager's own
        ``release``); the engine passes the runner's ``finish``, so that whatever the runner does with pages that
        come back (its ``poison_freed_pages``) also holds for requests that finish or are pushed out here."""
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
        self.release = release if release is not None else cache.release
        self.waiting: deque[Sequence] = deque()       # arrival order; the head may hold pages already (a prompt under way)
        self.running: deque[Sequence] = deque()       # requests whose prompt is in the cache
        self.waiting_since: dict[int, float] = {}
        self.num_preemptions = 0
        self.num_recomputed_tokens = 0

    # ------------------------------------------------------------------ intake
    def add(self, seq: Sequence) -> None:
        """Queues a request. What could never run is refused here: a request longer than the model allows or
        than all pages together (the reference finds out only when its scheduler stops making progress,
        scheduler.py:898-903)."""
        longest = seq.num_prompt_tokens + seq.max_tokens
        if longest > self.max_model_len:
            raise ValueError(f"prompt of {seq.num_prompt_tokens} tokens and max_tokens {seq.max_tokens} "
                             f"exceed max_model_len {self.max_model_len}")
        for g in self.cache.groups:
            if -(-longest // g.page_size) > g.num_pages:
                raise ValueError(f"a request of up to {longest} tokens needs {-(-longest // g.page_size)} pages; "
                                 f"the cache has {g.num_pages}")
        self._enqueue(seq)

    def is_finished(self) -> bool:
        return not self.waiting and not self.running

    def _enqueue(self, seq: Sequence) -> None:
        self.waiting.append(seq)
        self.waiting_since[seq.seq_id] = self.clock()

    # ------------------------------------------------------------------ the plan
    def schedule(self) -> SchedulePlan:
        plan = SchedulePlan()
        room = _Room(tokens=self.max_num_batched_tokens, requests=self.max_num_seqs)
        prompts_first = self.scheduler_policy == "prefill_first" and bool(self.waiting)
        overdue = self._head_is_overdue()
        if not prompts_first:
            # an overdue prompt finds one place and one token untouched by the decoding pass
            spare = 1 if overdue else 0
            self._decoding_pass(plan, _Room(room.tokens - spare, room.requests - spare))
            room = _Room(room.tokens - len(plan.decode_seqs), room.requests - len(plan.decode_seqs))
        self._admission_pass(plan, room, may_push_out=prompts_first or overdue)
        if plan.is_empty:
            raise RuntimeError("the scheduler cannot make progress: nothing can decode and the first waiting request "
                               "cannot be given a state slot and pages")
        return plan

    def _head_is_overdue(self) -> bool:
        if not self.waiting:
            return False
        now = self.clock()
        since = self.waiting_since.get(self.waiting[0].seq_id, now)
        return (now - since) * 1000.0 >= self.max_prefill_wait_ms

    def _decoding_pass(self, plan: SchedulePlan, room: _Room) -> None:
        """One token for every running request, in the queue's order, while the step has room. A request's newest
        token is stored by this step, at position ``num_tokens - 1``; where that starts a page, the page is
        taken now (scheduler.py:480-538)."""
        untouched: deque[Sequence] = deque()          # running requests that this pass has not reached or that stay out
        candidates, self.running = self.running, untouched
        while candidates:
            if not room.left:
                untouched.extend(candidates)          # no room for them in this step; they keep their places
                break
            seq = candidates.popleft()
            # whoever is pushed out to make room comes from those not yet planned (the rest of ``candidates``)
            while not self.cache.can_reserve(seq.seq_id, seq.num_tokens):
                loser = self._cheapest_to_recompute(candidates)
                if loser is None:
                    loser = seq                       # it is alone: it gives up its own pages and starts again
                else:
                    candidates.remove(loser)
                self._push_out(loser, plan)
                if loser is seq:
                    break
            else:
                self.cache.reserve(seq.seq_id, seq.num_tokens)
                seq.num_scheduled_tokens = seq.num_tokens - seq.num_cached_tokens      # always 1
                room.take(1)
                plan.decode_seqs.append(seq)
        # the planned requests keep their order at the front, whoever was not reached follows
        self.running = deque(plan.decode_seqs)
        self.running.extend(untouched)

    def _admission_pass(self, plan: SchedulePlan, room: _Room, may_push_out: bool) -> None:
        """The head of the waiting queue gets what the step has left (scheduler.py:579-884)."""
        while self.waiting and room.left:
            seq = self.waiting[0]
            if seq.seq_id not in self.cache and not self._admit(seq, plan, may_push_out):
                break                                  # first come, first served: nobody overtakes the head
            unfed = seq.num_tokens - seq.num_cached_tokens
            if unfed <= 0:
                raise RuntimeError(f"request {seq.seq_id} waits but has no tokens left to feed")
            seq.num_scheduled_tokens = min(unfed, room.tokens)
            room.take(seq.num_scheduled_tokens)
            plan.prefill_seqs.append(seq)
            if seq.num_scheduled_tokens == unfed:
                # its last portion: it decodes from the next step on
                seq.status = SequenceStatus.RUNNING
                self.waiting.popleft()
                self.waiting_since.pop(seq.seq_id, None)
                self.running.append(seq)
            else:
                self.waiting_since[seq.seq_id] = self.clock()       # it was served: its wait starts again

    def _admit(self, seq: Sequence, plan: SchedulePlan, may_push_out: bool) -> bool:
        """A new request needs a place among the live ones, a state slot, and pages for all the tokens it holds
        (prompt, and generated tokens of a request that is computed again), so that no later portion can run out
        of pages (nanovllm/engine/block_manager.py:696-749). ``may_push_out``: running requests that have no
        place in this step make room if need be. (Requests that this step already planned stay: the decoding ones
        and, unlike the reference, scheduler.py:674-719, the prompts just planned.)"""
        def fits() -> bool:
            live = len(self.running) + sum(1 for s in self.waiting if s.seq_id in self.cache)
            return live < self.max_num_seqs and self.cache.can_start(seq.token_ids)

        planned = {s.seq_id for s in plan.decode_seqs} | {s.seq_id for s in plan.prefill_seqs}
        while not fits():
            loser = self._cheapest_to_recompute(s for s in self.running if s.seq_id not in planned) if may_push_out else None
            if loser is None:
                return False
            self.running.remove(loser)
            self._push_out(loser, plan)
        self.cache.admit(seq.seq_id, seq.token_ids)
        self.cache.reserve(seq.seq_id, seq.num_tokens)
        # with shared prefixes the first pages may hold this request's first tokens already
        # (nanovllm/engine/block_manager.py:727-749)
        seq.num_cached_tokens = self.cache.num_tokens(seq.seq_id)
        return True

    @staticmethod
    def _cheapest_to_recompute(candidates) -> Sequence | None:
        """The request with the fewest tokens in the cache, the older one if two have as many
        (scheduler.py:350-378)."""
        return min(candidates, key=lambda s: (s.num_cached_tokens, s.seq_id), default=None)

    def _push_out(self, seq: Sequence, plan: SchedulePlan) -> None:
        """The request gives back all it holds and joins the waiting queue at the tail; all its tokens, generated
        ones included, are its prompt when its turn comes again (scheduler.py:906-949). The caller has taken it
        out of the running queue."""
        plan.preempted_seq_ids.append(seq.seq_id)
        self.num_preemptions += 1
        self.num_recomputed_tokens += seq.num_cached_tokens
        seq.status = SequenceStatus.WAITING
        seq.num_cached_tokens = 0
        seq.num_scheduled_tokens = 0
        if seq.seq_id in self.cache:
            self.release(seq.seq_id)
        self._enqueue(seq)

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
                self.release(seq.seq_id)
                self.running.remove(seq)
                finished.append(seq)
        return finished
