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


# ---- pages shared by their content -------------------------------------------------------------------------------

def shared(pages=12, page=4, slots=6):
    return CacheManager([PagedGroupSpec("all", page, pages)], slots, share_prefixes=True)


def feed(m, rid, tokens, upto=None):
    """Admits (if new) and stores ``tokens[:upto]``; returns how many of them were found in the cache."""
    upto = len(tokens) if upto is None else upto
    found = 0
    if rid not in m:
        m.admit(rid, tokens)
        found = m.num_tokens(rid)
    have = m.num_tokens(rid)
    m.reserve(rid, upto)
    m.commit(rid, upto, tokens[have:upto])
    m.check()
    return found


def test_a_known_start_is_taken_over_not_computed_again():
    m = shared()
    a = list(range(100, 114))                                   # 14 tokens: 3 full pages and a started one
    assert feed(m, "a", a) == 0
    ta = list(m.block_table("a"))
    b = a[:9] + [7, 7, 7]
    assert m.known_prefix(b) == ta[:2]
    assert feed(m, "b", b) == 8
    assert m.block_table("b")[:2] == ta[:2] and m.block_table("b")[2] not in ta
    assert m.holders[0][ta[0]] == 2 and m.holders[0][ta[2]] == 1
    free_before = m.num_free_pages()
    given_back = m.release("a")
    assert sorted(given_back[0]) == sorted(ta[2:]) and m.num_free_pages() == free_before + 2    # b still holds two
    m.check()
    # a free page keeps its content until it is handed out again: the third page comes back from the free list
    assert feed(m, "c", a) == 12
    assert m.block_table("c")[:3] == ta[:3]
    assert m.num_shared_tokens == 8 + 12
    m.release("b"), m.release("c")
    m.check()
    assert m.num_free_pages() == 12


def test_the_page_with_the_last_token_is_never_taken_over():
    m = shared()
    a = list(range(8))                                          # exactly two pages
    feed(m, "a", a)
    assert len(m.known_prefix(a)) == 1                          # one token at least is left to compute
    assert len(m.known_prefix(a + [1])) == 2
    assert m.known_prefix(a[:4]) == []
    assert feed(m, "b", a) == 4


def test_a_page_that_is_handed_out_again_forgets_its_content():
    m = shared(pages=4)
    a = list(range(50, 59))                                     # two full pages
    feed(m, "a", a)
    m.release("a")
    assert len(m.known_prefix(a)) == 2
    feed(m, "b", [1] * 16)                                      # takes all four pages
    assert m.known_prefix(a) == []
    assert all(tokens == (1, 1, 1, 1) for _, tokens in m.content.values())
    m.release("b")
    m.check()


def test_another_content_with_the_same_hash_is_not_taken(monkeypatch):
    import nanohybrid_vlm_amd.cache.manager as manager
    monkeypatch.setattr(manager, "chain_hash", lambda tokens, previous: 42)
    m = shared()
    feed(m, "a", [1, 2, 3, 4, 5])
    assert m.known_prefix([9, 9, 9, 9, 5]) == []
    assert len(m.known_prefix([1, 2, 3, 4, 5])) == 1


def test_sharing_needs_one_group_that_keeps_all_keys():
    with pytest.raises(ValueError, match="every layer keeps all keys"):
        CacheManager([PagedGroupSpec("w", 4, 8, window=5)], 2, share_prefixes=True)
    with pytest.raises(ValueError, match="every layer keeps all keys"):
        CacheManager([PagedGroupSpec("a", 4, 8), PagedGroupSpec("b", 4, 8)], 2, share_prefixes=True)
    m = shared()
    m.admit("a", [1, 2, 3])
    m.reserve("a", 3)
    with pytest.raises(CacheError, match="names the 3 tokens"):
        m.commit("a", 3)


@pytest.mark.parametrize("seed", range(8))
def test_random_orders_with_shared_pages(seed):
    """A stand-in for the device memory, one token per slot: whatever is shared, revived or handed out again,
    every live request finds its own tokens at its slots."""
    rng = random.Random(seed)
    ps = 4
    m = shared(pages=20, page=ps, slots=5)
    memory = {}
    starts = [[rng.randrange(50) for _ in range(rng.randint(3, 14))] for _ in range(3)]
    live, next_id = {}, 0                                        # id -> all its tokens
    for _ in range(700):
        op = rng.random()
        if op < 0.3:
            tokens = rng.choice(starts) + [rng.randrange(50) for _ in range(rng.randint(1, 12))]
            if m.can_start(tokens):
                m.admit(next_id, tokens)
                m.reserve(next_id, len(tokens))
                live[next_id] = tokens
                next_id += 1
            else:
                free = m.num_free_pages()
                in_use = sum(1 for p in m.known_prefix(tokens) if p in m.pools[0].used)
                assert not m.can_admit() or -(-len(tokens) // ps) - in_use > free
        elif op < 0.8 and live:
            rid = rng.choice(list(live))
            tokens, have = live[rid], m.num_tokens(rid)
            if have == len(tokens):                              # a generated token
                tokens.append(rng.randrange(50))
            upto = rng.randint(have + 1, len(tokens))
            if not m.can_reserve(rid, upto):
                continue
            m.reserve(rid, upto)
            table = m.block_table(rid)
            for p in range(have, upto):                          # the step stores the new tokens
                slot = table[p // ps] * ps + p % ps
                memory[slot] = tokens[p]
            m.commit(rid, upto, tokens[have:upto])
        elif live:
            rid = rng.choice(list(live))
            m.release(rid)
            del live[rid]
        m.check()
        for rid, tokens in live.items():
            table = m.block_table(rid)
            for p in range(m.num_tokens(rid)):
                assert memory[table[p // ps] * ps + p % ps] == tokens[p], "a request reads another's tokens"
    for rid in list(live):
        m.release(rid)
    m.check()
    assert m.num_free_pages() == 20 and m.num_shared_tokens > 0


def test_a_commit_can_be_taken_back():
    m = make(pages=8, page=4)
    m.admit("a")
    m.reserve("a", 6)
    m.commit("a", 5)
    m.reserve("a", 6)
    m.commit("a", 6)
    m.rewind("a", 5)                                        # the step that stored token 5 counts as not issued
    assert m.num_tokens("a") == 5 and len(m.block_table("a")) == 2
    m.commit("a", 6)
    with pytest.raises(CacheError):
        m.rewind("a", 7)
    m.check()
    with pytest.raises(CacheError):                         # a window's pages may be gone
        w = make(pages=6, page=4, window=6)
        w.admit("a"); w.reserve("a", 4); w.commit("a", 4)
        w.rewind("a", 3)
