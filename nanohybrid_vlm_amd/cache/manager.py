"""Book-keeping of the cache: pages, block tables and state slots. Pure CPU.

A model's cache units (one per entry of the model's run order that writes keys
and values) are sorted into *groups* by what they need: every key of the request
(``window=None``) or only the last ``window`` of them. Each group has a pool of
pages of its own and each request has one block table per group, so a page id
means the same place in every unit of its group.

Pages come from a first-in-first-out free list, as in the reference
(nanovllm/engine/block_manager.py:96-131): a page that is given back goes to the
tail and is handed out again only after all pages that were free before it, which
keeps page ids reproducible from run to run.

Beside the pages every live request holds one *state slot*: the index of its row
in pools of fixed-size per-request state (nanovllm/engine/hybrid_state.py:19-83).
An architecture without such state still gets slot ids; its pools are empty.
"""
from __future__ import annotations

from collections import deque
from dataclasses import dataclass, field
from typing import Hashable

NO_PAGE = -1


class CacheError(RuntimeError):
    """A request for pages or slots that breaks the manager's rules."""


class OutOfPages(CacheError):
    """Not enough free pages (or no free state slot) for what was asked."""


@dataclass(frozen=True)
class PagedGroupSpec:
    """One group of cache units with the same needs."""

    name: str
    page_size: int                  # tokens in a page
    num_pages: int                  # pages in this group's pool
    window: int | None = None       # None: all keys are kept; n: a query sees the last n keys (itself included)

    def __post_init__(self):
        if self.page_size <= 0:
            raise ValueError("page_size must be positive")
        if self.num_pages <= 0:
            raise ValueError("num_pages must be positive")
        if self.window is not None and self.window <= 0:
            raise ValueError("window must be positive")


class PageAllocator:
    """Free list and used set of one pool (block_manager.py:96-131)."""

    def __init__(self, num_pages: int):
        self.num_pages = num_pages
        self.free: deque[int] = deque(range(num_pages))
        self.used: set[int] = set()

    @property
    def num_free(self) -> int:
        return len(self.free)

    def take(self) -> int:
        if not self.free:
            raise OutOfPages("no free page")
        page = self.free.popleft()
        self.used.add(page)
        return page

    def give_back(self, page: int) -> None:
        if page not in self.used:
            raise CacheError(f"page {page} is given back but is not in use")
        self.used.remove(page)
        self.free.append(page)


class StateSlotAllocator:
    """Row numbers of the per-request state pools (hybrid_state.py:19-83)."""

    def __init__(self, num_slots: int):
        if num_slots <= 0:
            raise ValueError("num_slots must be positive")
        self.num_slots = num_slots
        self.free: deque[int] = deque(range(num_slots))
        self.used: set[int] = set()

    def can_allocate(self) -> bool:
        return bool(self.free)

    def allocate(self) -> int:
        if not self.free:
            raise OutOfPages("no free state slot")
        slot = self.free.popleft()
        self.used.add(slot)
        return slot

    def release(self, slot: int) -> None:
        if slot not in self.used:
            raise CacheError(f"state slot {slot} is released but is not in use")
        self.used.remove(slot)
        self.free.append(slot)


@dataclass
class RequestCache:
    """What one live request holds."""

    state_slot: int
    num_tokens: int = 0                                   # tokens whose keys and values are stored
    tables: list[list[int]] = field(default_factory=list)  # per group: logical page -> page id or NO_PAGE
    first_live: list[int] = field(default_factory=list)   # per group: first logical page not yet given back


class CacheManager:
    """Pages and slots of all live requests.

    The life of a request: ``admit`` (takes a state slot), then any number of
    ``reserve(new_len)`` (pages for positions below ``new_len``) each followed,
    after the step that stored those tokens, by ``commit(new_len)`` (which also
    gives back pages that a window has passed), and ``release`` at the end.
    """

    def __init__(self, groups: list[PagedGroupSpec], num_state_slots: int):
        if not groups:
            raise ValueError("at least one paged group is needed")
        self.groups = list(groups)
        self.pools = [PageAllocator(g.num_pages) for g in groups]
        self.slots = StateSlotAllocator(num_state_slots)
        self.requests: dict[Hashable, RequestCache] = {}

    # ---- questions ----------------------------------------------------
    def __contains__(self, request_id) -> bool:
        return request_id in self.requests

    def num_tokens(self, request_id) -> int:
        return self.requests[request_id].num_tokens

    def state_slot(self, request_id) -> int:
        return self.requests[request_id].state_slot

    def block_table(self, request_id, group: int = 0) -> list[int]:
        return self.requests[request_id].tables[group]

    def num_free_pages(self, group: int = 0) -> int:
        return self.pools[group].num_free

    def pages_needed(self, request_id, new_len: int) -> list[int]:
        """Pages that ``reserve(request_id, new_len)`` would take, per group.
        ``request_id`` may be unknown (a request not yet admitted)."""
        rc = self.requests.get(request_id)
        out = []
        for gi, g in enumerate(self.groups):
            have = len(rc.tables[gi]) if rc is not None else 0
            out.append(max(0, -(-new_len // g.page_size) - have))
        return out

    def can_admit(self) -> bool:
        return self.slots.can_allocate()

    def can_reserve(self, request_id, new_len: int) -> bool:
        need = self.pages_needed(request_id, new_len)
        return all(n <= p.num_free for n, p in zip(need, self.pools))

    # ---- actions ------------------------------------------------------
    def admit(self, request_id) -> int:
        if request_id in self.requests:
            raise CacheError(f"request {request_id!r} is already live")
        slot = self.slots.allocate()
        self.requests[request_id] = RequestCache(
            state_slot=slot,
            tables=[[] for _ in self.groups],
            first_live=[0 for _ in self.groups],
        )
        return slot

    def reserve(self, request_id, new_len: int) -> None:
        """Make sure pages exist for every position below ``new_len``.
        Takes all of them or, when a pool is short, none (``OutOfPages``)."""
        rc = self.requests[request_id]
        if new_len < rc.num_tokens:
            raise CacheError(f"request {request_id!r}: cannot shrink from {rc.num_tokens} to {new_len} tokens")
        need = self.pages_needed(request_id, new_len)
        for gi, n in enumerate(need):
            if n > self.pools[gi].num_free:
                raise OutOfPages(
                    f"group '{self.groups[gi].name}': {n} pages needed for request {request_id!r}, "
                    f"{self.pools[gi].num_free} free")
        for gi, n in enumerate(need):
            for _ in range(n):
                rc.tables[gi].append(self.pools[gi].take())

    def commit(self, request_id, new_len: int) -> None:
        """The step that stored the tokens below ``new_len`` has been issued.
        Pages of a windowed group whose every key lies before the window of the
        next query (position ``new_len``) are given back."""
        rc = self.requests[request_id]
        if new_len < rc.num_tokens:
            raise CacheError(f"request {request_id!r}: commit of {new_len} below {rc.num_tokens}")
        for gi, g in enumerate(self.groups):
            if new_len > len(rc.tables[gi]) * g.page_size:
                raise CacheError(f"request {request_id!r}: commit of {new_len} tokens beyond its reserved pages")
        rc.num_tokens = new_len
        for gi, g in enumerate(self.groups):
            if g.window is None:
                continue
            first_needed = new_len - g.window + 1          # oldest key the next query sees
            if first_needed <= 0:
                continue
            passed = first_needed // g.page_size           # logical pages wholly before it
            table = rc.tables[gi]
            for lp in range(rc.first_live[gi], min(passed, len(table))):
                self.pools[gi].give_back(table[lp])
                table[lp] = NO_PAGE
            rc.first_live[gi] = max(rc.first_live[gi], min(passed, len(table)))

    def release(self, request_id) -> None:
        """Give back everything the request holds (block_manager.py:751-802:
        pages go back in reverse order)."""
        rc = self.requests.pop(request_id, None)
        if rc is None:
            raise CacheError(f"request {request_id!r} is released but is not live")
        for gi, table in enumerate(rc.tables):
            for page in reversed(table):
                if page != NO_PAGE:
                    self.pools[gi].give_back(page)
        self.slots.release(rc.state_slot)

    # ---- self-check (tests call it after every operation) ---------------
    def check(self) -> None:
        for gi, pool in enumerate(self.pools):
            free = list(pool.free)
            if len(set(free)) != len(free):
                raise AssertionError(f"group {gi}: a page is twice in the free list")
            if set(free) & pool.used:
                raise AssertionError(f"group {gi}: a page is both free and in use")
            if len(free) + len(pool.used) != pool.num_pages:
                raise AssertionError(f"group {gi}: pages lost: {len(free)} free + {len(pool.used)} used != {pool.num_pages}")
            held = [p for rc in self.requests.values() for p in rc.tables[gi] if p != NO_PAGE]
            if len(set(held)) != len(held):
                raise AssertionError(f"group {gi}: a page is held twice")
            if set(held) != pool.used:
                raise AssertionError(f"group {gi}: held pages and used set differ")
        slots = [rc.state_slot for rc in self.requests.values()]
        if len(set(slots)) != len(slots) or set(slots) != self.slots.used:
            raise AssertionError("state slots of live requests and used set differ")
        if len(self.slots.free) + len(self.slots.used) != self.slots.num_slots:
            raise AssertionError("state slots lost")
