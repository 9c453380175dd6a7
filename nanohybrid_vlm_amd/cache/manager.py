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

With ``share_prefixes`` a full page is also known by its content: a hash over its
tokens chained to the hash of the page before it (block_manager.py:102-108). A new
request whose first pages have known contents takes those pages instead of
computing them again; a page then has several holders and goes back to the free
list when the last one lets go. A free page keeps its content until it is handed
out again, so a request that was pushed out finds its own pages again
(block_manager.py:110-119, 727-749).

Beside the pages every live request holds one *state slot*: the index of its row
in pools of fixed-size per-request state (nanovllm/engine/hybrid_state.py:19-83).
An architecture without such state still gets slot ids; its pools are empty.
"""
from __future__ import annotations

import hashlib
import struct
from collections import deque
from dataclasses import dataclass, field
from typing import Hashable, Sequence

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

    def revive(self, page: int) -> None:
        """Takes one particular free page (its content is wanted again)."""
        if page in self.used:
            raise CacheError(f"page {page} is revived but is in use")
        self.free.remove(page)
        self.used.add(page)


def chain_hash(tokens: Sequence[int], previous: int | None) -> int:
    """Hash of one full page: its tokens and the hash of the page before it, so that equal hashes mean equal
    prefixes (block_manager.py:102-108 chains xxh64 the same way; the function itself is free to differ,
    since hashes never leave the process)."""
    h = hashlib.blake2b(digest_size=8)
    if previous is not None:
        h.update(previous.to_bytes(8, "little"))
    h.update(struct.pack(f"<{len(tokens)}q", *tokens))
    return int.from_bytes(h.digest(), "little")


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
    # with shared prefixes only
    tokens: list[int] = field(default_factory=list)        # the tokens below num_tokens
    num_hashed: int = 0                                    # leading pages whose chain hash is known
    last_hash: int | None = None                           # chain hash of page num_hashed - 1


class CacheManager:
    """Pages and slots of all live requests.

    The life of a request: ``admit`` (takes a state slot), then any number of
    ``reserve(new_len)`` (pages for positions below ``new_len``) each followed,
    after the step that stored those tokens, by ``commit(new_len)`` (which also
    gives back pages that a window has passed), and ``release`` at the end.
    """

    def __init__(self, groups: list[PagedGroupSpec], num_state_slots: int, share_prefixes: bool = False):
        if not groups:
            raise ValueError("at least one paged group is needed")
        if share_prefixes and (len(groups) != 1 or groups[0].window is not None):
            # a page of a windowed group does not stay, and a second group would need the same hits
            raise ValueError("prefixes can be shared only when every layer keeps all keys (one group, no window)")
        self.groups = list(groups)
        self.pools = [PageAllocator(g.num_pages) for g in groups]
        self.slots = StateSlotAllocator(num_state_slots)
        self.requests: dict[Hashable, RequestCache] = {}
        self.share_prefixes = share_prefixes
        self.holders: list[dict[int, int]] = [{} for _ in groups]      # per group: page -> number of requests holding it
        self.content: dict[int, tuple[int, tuple[int, ...]]] = {}      # page -> (chain hash, its tokens)
        self.page_of_hash: dict[int, int] = {}
        self.num_shared_tokens = 0                                     # tokens that requests did not have to compute

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

    def num_free_slots(self) -> int:
        return len(self.slots.free)

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

    def known_prefix(self, tokens: Sequence[int]) -> list[int]:
        """The pages that hold the start of ``tokens`` already, in order. The page with the last token is
        never among them, so a request always has a token left to compute (block_manager.py:711-725)."""
        if not self.share_prefixes:
            return []
        ps = self.groups[0].page_size
        pages, h = [], None
        for lp in range((len(tokens) - 1) // ps):
            chunk = tuple(tokens[lp * ps:(lp + 1) * ps])
            h = chain_hash(chunk, h)
            page = self.page_of_hash.get(h)
            if page is None or self.content[page][1] != chunk:      # unknown, or another content with this hash
                break
            pages.append(page)
        return pages

    def can_start(self, tokens: Sequence[int]) -> bool:
        """Whether a new request with these tokens can be admitted and given pages for all of them now."""
        if not self.slots.can_allocate():
            return False
        if not self.share_prefixes:
            return self.can_reserve(None, len(tokens))
        g, pool = self.groups[0], self.pools[0]
        in_use = sum(1 for p in self.known_prefix(tokens) if p in pool.used)
        return -(-len(tokens) // g.page_size) - in_use <= pool.num_free

    def _has_pages(self, rc: RequestCache, new_len: int) -> bool:
        """Whether the request's tables already reach ``new_len`` (the usual case of a decoding step)."""
        for g, table in zip(self.groups, rc.tables):
            if len(table) * g.page_size < new_len:
                return False
        return True

    def can_reserve(self, request_id, new_len: int) -> bool:
        rc = self.requests.get(request_id)
        if rc is not None and self._has_pages(rc, new_len):
            return True
        need = self.pages_needed(request_id, new_len)
        return all(n <= p.num_free for n, p in zip(need, self.pools))

    # ---- actions ------------------------------------------------------
    def admit(self, request_id, tokens: Sequence[int] | None = None) -> int:
        """Takes a state slot. With shared prefixes and the request's ``tokens``, the pages that hold their
        start already become the request's first pages, and ``num_tokens(request_id)`` says how many tokens
        need not be computed (block_manager.py:727-749)."""
        if request_id in self.requests:
            raise CacheError(f"request {request_id!r} is already live")
        hits = self.known_prefix(tokens) if tokens is not None else []
        slot = self.slots.allocate()
        rc = RequestCache(state_slot=slot, tables=[[] for _ in self.groups], first_live=[0 for _ in self.groups])
        self.requests[request_id] = rc
        if hits:
            pool, holders, ps = self.pools[0], self.holders[0], self.groups[0].page_size
            for page in hits:
                if page not in pool.used:
                    pool.revive(page)
                holders[page] = holders.get(page, 0) + 1
                rc.tables[0].append(page)
            rc.num_tokens = len(hits) * ps
            rc.tokens = list(tokens[:rc.num_tokens])
            rc.num_hashed = len(hits)
            rc.last_hash = self.content[hits[-1]][0]
            self.num_shared_tokens += rc.num_tokens
        return slot

    def _take(self, gi: int) -> int:
        page = self.pools[gi].take()
        known = self.content.pop(page, None)        # its old content is about to be overwritten
        if known is not None and self.page_of_hash.get(known[0]) == page:
            del self.page_of_hash[known[0]]
        self.holders[gi][page] = 1
        return page

    def _let_go(self, gi: int, page: int) -> bool:
        """One holder less; True if the page went back to the free list."""
        left = self.holders[gi][page] - 1
        if left:
            self.holders[gi][page] = left
            return False
        del self.holders[gi][page]
        self.pools[gi].give_back(page)
        return True

    def reserve(self, request_id, new_len: int) -> None:
        """Make sure pages exist for every position below ``new_len``.
        Takes all of them or, when a pool is short, none (``OutOfPages``)."""
        rc = self.requests[request_id]
        if new_len < rc.num_tokens:
            raise CacheError(f"request {request_id!r}: cannot shrink from {rc.num_tokens} to {new_len} tokens")
        if self._has_pages(rc, new_len):
            return
        need = self.pages_needed(request_id, new_len)
        for gi, n in enumerate(need):
            if n > self.pools[gi].num_free:
                raise OutOfPages(
                    f"group '{self.groups[gi].name}': {n} pages needed for request {request_id!r}, "
                    f"{self.pools[gi].num_free} free")
        for gi, n in enumerate(need):
            for _ in range(n):
                rc.tables[gi].append(self._take(gi))

    def commit(self, request_id, new_len: int, new_tokens: Sequence[int] | None = None) -> list[list[int]]:
        """The step that stored the tokens below ``new_len`` has been issued.
        Pages of a windowed group whose every key lies before the window of the
        next query (position ``new_len``) are given back. Returns the pages given
        back, per group. With shared prefixes ``new_tokens`` are the tokens that
        the step stored; pages that they filled become known by their content
        (block_manager.py:811-825)."""
        rc = self.requests[request_id]
        if new_len < rc.num_tokens:
            raise CacheError(f"request {request_id!r}: commit of {new_len} below {rc.num_tokens}")
        for gi, g in enumerate(self.groups):
            if new_len > len(rc.tables[gi]) * g.page_size:
                raise CacheError(f"request {request_id!r}: commit of {new_len} tokens beyond its reserved pages")
        if self.share_prefixes and new_len > rc.num_tokens:
            if new_tokens is None or len(new_tokens) != new_len - rc.num_tokens:
                raise CacheError(f"request {request_id!r}: with shared prefixes a commit names the "
                                 f"{new_len - rc.num_tokens} tokens that were stored")
            rc.tokens.extend(new_tokens)
            ps, table = self.groups[0].page_size, rc.tables[0]
            for lp in range(rc.num_hashed, new_len // ps):
                chunk = tuple(rc.tokens[lp * ps:(lp + 1) * ps])
                rc.last_hash = chain_hash(chunk, rc.last_hash)
                if rc.last_hash not in self.page_of_hash:           # the first page with this content stays the known one
                    self.page_of_hash[rc.last_hash] = table[lp]
                    self.content[table[lp]] = (rc.last_hash, chunk)
            rc.num_hashed = max(rc.num_hashed, new_len // ps)
        rc.num_tokens = new_len
        given_back: list[list[int]] = [[] for _ in self.groups]
        for gi, g in enumerate(self.groups):
            if g.window is None:
                continue
            first_needed = new_len - g.window + 1          # oldest key the next query sees
            if first_needed <= 0:
                continue
            passed = first_needed // g.page_size           # logical pages wholly before it
            table = rc.tables[gi]
            for lp in range(rc.first_live[gi], min(passed, len(table))):
                if self._let_go(gi, table[lp]):
                    given_back[gi].append(table[lp])
                table[lp] = NO_PAGE
            rc.first_live[gi] = max(rc.first_live[gi], min(passed, len(table)))
        return given_back

    def rewind(self, request_id, new_len: int) -> None:
        """Takes a commit back: the tokens from ``new_len`` on count as not stored (a step that was issued ahead of
        its turn and is run again). Pages stay reserved. Not with windows (their pages may be gone) and not with
        shared prefixes (pages may have become known by a content that is taken back)."""
        rc = self.requests[request_id]
        if self.share_prefixes or any(g.window is not None for g in self.groups):
            raise CacheError("rewind: not with windows or shared prefixes")
        if not 0 <= new_len <= rc.num_tokens:
            raise CacheError(f"request {request_id!r}: rewind to {new_len} from {rc.num_tokens}")
        rc.num_tokens = new_len

    def release(self, request_id) -> list[list[int]]:
        """Give back everything the request holds (block_manager.py:751-802:
        pages go back in reverse order). Returns the pages given back, per group."""
        rc = self.requests.pop(request_id, None)
        if rc is None:
            raise CacheError(f"request {request_id!r} is released but is not live")
        given_back: list[list[int]] = [[] for _ in self.groups]
        for gi, table in enumerate(rc.tables):
            for page in reversed(table):
                if page != NO_PAGE and self._let_go(gi, page):
                    given_back[gi].append(page)
        self.slots.release(rc.state_slot)
        return given_back

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
            if not self.share_prefixes and len(set(held)) != len(held):
                raise AssertionError(f"group {gi}: a page is held twice")
            if set(held) != pool.used:
                raise AssertionError(f"group {gi}: held pages and used set differ")
            counts: dict[int, int] = {}
            for p in held:
                counts[p] = counts.get(p, 0) + 1
            if counts != self.holders[gi]:
                raise AssertionError(f"group {gi}: holder counts differ from the block tables")
            for rc in self.requests.values():
                own = [p for p in rc.tables[gi] if p != NO_PAGE]
                if len(set(own)) != len(own):
                    raise AssertionError(f"group {gi}: a request holds a page twice")
        for h, page in self.page_of_hash.items():
            if page not in self.content or self.content[page][0] != h:
                raise AssertionError("a hash points at a page with another content")
        for rc in self.requests.values():
            if self.share_prefixes and len(rc.tokens) != rc.num_tokens:
                raise AssertionError("a request's tokens and its token count differ")
        slots = [rc.state_slot for rc in self.requests.values()]
        if len(set(slots)) != len(slots) or set(slots) != self.slots.used:
            raise AssertionError("state slots of live requests and used set differ")
        if len(self.slots.free) + len(self.slots.used) != self.slots.num_slots:
            raise AssertionError("state slots lost")
