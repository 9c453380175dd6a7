"""The cache manager's book-keeping: no page lost, held twice or freed twice, under
random orders of requests; FIFO reuse; windows; state slots."""
import random

import pytest

from nanohybrid_vlm_amd.cache.manager import (NO_PAGE, CacheError, CacheManager, OutOfPages, PagedGroupSpec,
                                              StateSlotAllocator)


def make(pages=8, page=4, window=None, slots=4, extra_group=None):
    groups = [PagedGroupSpec("all", page, pages)]
    if extra_group:
        groups.append(extra_group)
    if window:
        groups = [PagedGroupSpec("w", page, pages, window)]
    return CacheManager(groups, slots)


def test_pages_come_first_in_first_out_and_are_used_again():
    m = make(pages=4, page=4)
    m.admit("a"); m.reserve("a", 9); m.commit("a", 9)
    assert m.block_table("a") == [0, 1, 2]
    m.admit("b"); m.reserve("b", 1)
    assert m.block_table("b") == [3]
    with pytest.raises(OutOfPages):
        m.reserve("b", 5)
    assert m.block_table("b") == [3], "a failed reserve takes nothing"
    m.release("a")                               # pages go back in reverse: 2, 1, 0
    m.reserve("b", 16)
    assert m.block_table("b") == [3, 2, 1, 0]
    m.check()


def test_reserve_is_idempotent_and_commit_is_bounded():
    m = make()
    m.admit(1)
    m.reserve(1, 6); m.reserve(1, 6); m.reserve(1, 5)
    assert len(m.block_table(1)) == 2
    with pytest.raises(CacheError, match="beyond"):
        m.commit(1, 9)
    m.commit(1, 6)
    with pytest.raises(CacheError, match="below|shrink"):
        m.reserve(1, 3)
    assert m.num_tokens(1) == 6


def test_double_actions_are_errors():
    m = make()
    m.admit("a")
    with pytest.raises(CacheError, match="already"):
        m.admit("a")
    m.release("a")
    with pytest.raises(CacheError, match="not live"):
        m.release("a")
    s = StateSlotAllocator(2)
    a = s.allocate(); s.release(a)
    with pytest.raises(CacheError):
        s.release(a)


def test_state_slots_are_unique_and_run_out():
    m = make(slots=2)
    assert m.admit("a") == 0 and m.admit("b") == 1
    assert not m.can_admit()
    with pytest.raises(OutOfPages, match="slot"):
        m.admit("c")
    m.release("a")
    assert m.admit("c") == 0
    m.check()


def test_window_gives_pages_back_when_passed():
    m = make(pages=6, page=4, window=6)
    m.admit("a")
    m.reserve("a", 10); m.commit("a", 10)
    # the next query (position 10) sees keys 5..10: page 0 (keys 0..3) has been passed, page 1 (4..7) not
    assert m.block_table("a") == [NO_PAGE, 1, 2]
    assert m.num_free_pages() == 4
    m.reserve("a", 13); m.commit("a", 13)       # next query 13 sees 8..13: page 1 passed too
    assert m.block_table("a")[:2] == [NO_PAGE, NO_PAGE] and len(m.block_table("a")) == 4
    m.check()
    m.release("a")
    assert m.num_free_pages() == 6
    m.check()


def test_groups_have_pools_of_their_own():
    m = make(pages=8, page=4, extra_group=PagedGroupSpec("w", 4, 3, window=4))
    m.admit("a")
    assert m.pages_needed("a", 9) == [3, 3]
    m.reserve("a", 9); m.commit("a", 9)
    assert m.num_free_pages(0) == 5
    assert m.num_free_pages(1) == 1              # window 4 at length 9: keys 6..9 -> page 0 passed
    assert not m.can_reserve("a", 20)            # the small pool is the limit
    m.check()


@pytest.mark.parametrize("seed", range(8))
@pytest.mark.parametrize("window", [None, 5])
def test_random_orders_keep_the_invariants(seed, window):
    rng = random.Random(seed)
    groups = [PagedGroupSpec("g0", 4, 24, window)]
    if seed % 2:
        groups.append(PagedGroupSpec("g1", 4, 16, 7))
    m = CacheManager(groups, num_state_slots=5)
    live, next_id = {}, 0
    for _ in range(600):
        op = rng.random()
        if op < 0.25 and m.can_admit():
            m.admit(next_id); live[next_id] = 0; next_id += 1
        elif op < 0.8 and live:
            rid = rng.choice(list(live))
            new_len = live[rid] + rng.randint(1, 9)
            if m.can_reserve(rid, new_len):
                m.reserve(rid, new_len); m.commit(rid, new_len); live[rid] = new_len
            else:
                with pytest.raises(OutOfPages):
                    m.reserve(rid, new_len)
        elif live:
            rid = rng.choice(list(live))
            m.release(rid); del live[rid]
        m.check()
        for rid, n in live.items():
            for gi, g in enumerate(m.groups):
                table = m.block_table(rid, gi)
                assert len(table) >= -(-n // g.page_size)
                first_needed = 0 if g.window is None else max(0, n - g.window + 1)
                for lp in range(first_needed // g.page_size, -(-n // g.page_size)):
                    assert table[lp] != NO_PAGE, "a page that the next query reads was given back"
    for rid in list(live):
        m.release(rid)
    m.check()
    assert all(m.num_free_pages(gi) == g.num_pages for gi, g in enumerate(m.groups))
