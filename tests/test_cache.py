"""The cache manager on the host: no page is lost, held twice or freed twice, under random
orders of requests; windows give pages back; freed pages are used again in order; prefix
hashes; state slots."""
import random
from types import SimpleNamespace

import pytest

from nano_vllm_amd.cache import (CacheGroup, CacheManager, OutOfPages, PageError, PagePool, SlotPool, chain_hash,
                                 plan_groups)
from nano_vllm_amd.parts.spec import FixedState, PagedKV


def _manager(pages=8, page=4, groups=(None,), slots=0, prefix=True):
    gs = [CacheGroup(w, (i,)) for i, w in enumerate(groups)]
    return CacheManager(gs, page, pages, num_state_slots=slots, has_state=slots > 0, enable_prefix_caching=prefix)


def test_plan_groups_by_need():
    needs = [PagedKV(2, 16), PagedKV(2, 16, window=8), None, PagedKV(4, 32), FixedState({"s": ((3,), "float32")}),
             PagedKV(2, 16, window=8), PagedKV(2, 16, window=32)]
    groups, state = plan_groups(needs)
    assert [(g.window, g.runs) for g in groups] == [(None, (0, 3)), (8, (1, 5)), (32, (6,))]
    assert state == [4]


def test_pages_are_taken_and_given_back():
    m = _manager(pages=4, page=4)
    m.admit("a")
    m.reserve("a", 5)
    assert m.table("a", 0) == [0, 1] and m.pools[0].num_free == 2
    m.reserve("a", 8)                                  # the same two pages suffice
    assert m.table("a", 0) == [0, 1]
    m.reserve("a", 9)
    assert m.table("a", 0) == [0, 1, 2]
    m.check()
    m.release("a")
    assert m.pools[0].num_free == 4
    m.check()


def test_freed_pages_are_used_again_oldest_first_and_tails_before_heads():
    m = _manager(pages=4, page=2)
    m.admit("a"); m.reserve("a", 6)                    # pages 0 1 2
    m.release("a")                                     # freed in the order 2 1 0, behind the never-used 3
    m.admit("b"); m.reserve("b", 8)
    assert m.table("b", 0) == [3, 2, 1, 0]             # block_manager.py:43-56,94-101


def test_out_of_pages_leaves_the_request_as_it_was():
    m = _manager(pages=3, page=4)
    m.admit("a"); m.reserve("a", 8)
    m.admit("b")
    assert not m.can_reserve("b", 8)
    with pytest.raises(OutOfPages):
        m.reserve("b", 8)
    assert m.table("b", 0) == [] and m.pools[0].num_free == 1
    m.check()
    m.reserve("b", 4)
    m.check()


def test_freeing_twice_is_an_error():
    pool = PagePool(2, 4)
    p = pool.take()
    pool.give_back(p)
    with pytest.raises(PageError):
        pool.give_back(p)
    m = _manager()
    m.admit("a")
    m.release("a")
    with pytest.raises(KeyError):
        m.release("a")
    m.admit("b")
    with pytest.raises(PageError):
        m.admit("b")


def test_window_gives_passed_pages_back():
    m = _manager(pages=4, page=4, groups=(None, 6))
    m.admit("a")
    pos = 0
    for n in (5, 3, 4, 1, 1, 1, 1):                     # portions, then single tokens
        m.reserve("a", pos + n, first_query=pos)
        pos += n
        full, win = m.table("a", 0), m.table("a", 1)
        assert all(p >= 0 for p in full) and len(full) == (pos + 3) // 4
        first_needed = max(0, (pos - n) - 6 + 1) // 4   # oldest key the step's first query reads
        assert all(p == -1 for p in win[:first_needed]) and all(p >= 0 for p in win[first_needed:])
        m.check()
    assert m.table("a", 1)[:2] == [-1, -1]
    assert m.pools[1].num_free == 4 - 2
    m.release("a")
    m.check()
    assert m.pools[0].num_free == 4 and m.pools[1].num_free == 4


def test_window_group_lets_a_long_request_live_on_few_pages():
    m = _manager(pages=3, page=4, groups=(8,))
    m.admit("a")
    for pos in range(0, 100):
        m.reserve("a", pos + 1, first_query=pos)        # never more than 3 pages held
        m.check()
    assert sum(1 for p in m.table("a", 0) if p >= 0) <= 3


@pytest.mark.parametrize("seed", range(6))
def test_random_orders_never_lose_or_double_a_page(seed):
    rng = random.Random(seed)
    m = _manager(pages=24, page=4, groups=(None, 10), slots=6, prefix=False)
    live = {}
    for step in range(600):
        op = rng.random()
        if op < 0.25 and len(live) < 6:
            rid = f"r{step}"
            m.admit(rid)
            live[rid] = 0
        elif op < 0.85 and live:
            rid = rng.choice(list(live))
            n = rng.choice([1, 1, 1, 2, 3, 7, 12])
            new_len = live[rid] + n
            if m.can_reserve(rid, new_len, first_query=live[rid]):
                m.reserve(rid, new_len, first_query=live[rid])
                live[rid] = new_len
            else:
                with pytest.raises(OutOfPages):
                    m.reserve(rid, new_len, first_query=live[rid])
        elif live:
            rid = rng.choice(list(live))
            m.release(rid)
            del live[rid]
        m.check()
        for rid, n in live.items():
            assert len(m.table(rid, 0)) == (n + 3) // 4
    for rid in list(live):
        m.release(rid)
    m.check()
    assert all(pool.num_free == pool.num_pages for pool in m.pools) and m.slots.num_free == 6


# ------------------------------------------------------------------------------ prefix hashes
def test_chain_hash_depends_on_the_prefix():
    a = chain_hash([1, 2, 3, 4])
    assert a == chain_hash([1, 2, 3, 4]) and a != chain_hash([1, 2, 3, 5])
    assert chain_hash([5, 6, 7, 8], a) != chain_hash([5, 6, 7, 8])


def test_prefix_pages_are_found_and_shared_but_never_the_last():
    m = _manager(pages=8, page=4)
    toks = list(range(10, 22))                         # 12 tokens = 3 full pages
    assert m.can_admit(toks) == 0
    assert m.admit_with_prefix("a", toks) == 0
    m.register_full_pages("a", toks, 12)
    # an equal prompt: the first two pages are shared, the last one is computed again (block_manager.py:62)
    assert m.can_admit(toks) == 2
    assert m.admit_with_prefix("b", toks) == 8
    assert m.table("b", 0)[:2] == m.table("a", 0)[:2] and m.table("b", 0)[2] != m.table("a", 0)[2]
    assert m.pools[0].ref_count[m.table("a", 0)[0]] == 2
    m.check()
    # a prompt that differs inside the second page shares only the first
    other = toks[:5] + [99] + toks[6:]
    assert m.can_admit(other) == 1
    m.release("a")
    m.check()
    assert m.pools[0].ref_count[m.table("b", 0)[0]] == 1
    m.release("b")
    m.check()
    # freed pages stay findable until they are taken again (block_manager.py:43-51)
    assert m.can_admit(toks + [1]) == 3
    assert m.admit_with_prefix("c", toks + [1]) == 12
    m.check()


def test_a_hit_needs_equal_tokens_not_only_an_equal_hash():
    m = _manager(pages=4, page=2)
    m.admit_with_prefix("a", [1, 2, 3])
    m.register_full_pages("a", [1, 2, 3], 3)
    page = m.table("a", 0)[0]
    m.pools[0].tokens_of[page] = (7, 7)                 # as after a hash collision
    assert m.can_admit([1, 2, 3]) == 0


def test_a_hit_on_a_free_page_still_takes_it():
    m = _manager(pages=4, page=2)
    toks = [1, 2, 3, 4, 5]
    m.admit_with_prefix("a", toks)
    m.register_full_pages("a", toks, 5)
    m.release("a")                                      # free list: 3 (never used), then a's 2, 1, 0
    m.admit("x"); m.reserve("x", 2)                     # takes page 3
    assert m.can_admit(toks) == 2                       # both hashed pages are still there, free: 3 free pages suffice
    m.admit("y"); m.reserve("y", 2)                     # takes a's unhashed tail page
    assert m.can_admit(toks) == -1                      # 3 pages wanted, hits are free pages themselves: 2 free < 3
    assert m.can_admit(toks[:4]) == 1                   # 2 pages wanted, 2 free (one of them the hit)
    m.check()


def test_prefix_caching_is_off_with_state_only():
    assert _manager(groups=(None, 8)).prefix_caching is True
    assert _manager(groups=(8,)).prefix_caching is True
    assert _manager(slots=2).prefix_caching is False
    assert _manager(prefix=False).prefix_caching is False
    assert _manager().prefix_caching is True


def test_prefix_pages_of_a_window_group():
    """An all-keys group beside a window of 6 keys, pages of 4: a request that starts at page n
    looks back at positions 4n - 5 .. 4n - 1, so the window group has to stand for pages n - 2
    and n - 1 only, and its earlier entries stay -1."""
    m = _manager(pages=12, page=4, groups=(None, 6))
    toks = list(range(100, 122))                        # 22 tokens: 5 full pages and two tokens
    assert m.admit_with_prefix("a", toks) == 0
    for done in (8, 16, 22):                            # in three steps, as portions of a prompt
        m.reserve("a", 22, first_query=done - 8 if done < 22 else 16)
        m.register_full_pages("a", toks, done)
        m.check()
    ta, wa = list(m.table("a", 0)), list(m.table("a", 1))
    assert wa[:2] == [-1, -1] and all(p >= 0 for p in wa[2:])      # pages 0 and 1 were passed at position 16
    # an equal prompt: five pages are left out; the window group shares pages 3 and 4
    hits, pages = m.match_prefix(toks)
    assert hits == 5 and pages[0] == ta[:5] and pages[1] == [-1, -1, -1, wa[3], wa[4]]
    assert m.admit_with_prefix("b", toks) == 20
    assert m.table("b", 0)[:5] == ta[:5] and m.table("b", 1)[:5] == [-1, -1, -1, wa[3], wa[4]]
    assert m.pools[1].ref_count[wa[4]] == 2 and m.pools[1].ref_count[wa[2]] == 1
    m.check()
    m.release("a")
    m.check()
    assert m.pools[1].ref_count[wa[4]] == 1
    m.release("b")
    m.check()
    assert all(pool.num_free == pool.num_pages for pool in m.pools)
    # the pages that a's window had passed went back first and are findable still
    # (nothing has taken them): a prompt cut after two pages finds both groups' pages 0 and 1
    assert m.can_admit(toks[:9]) == 2


def test_a_window_page_that_is_gone_shortens_the_hit():
    m = _manager(pages=12, page=4, groups=(None, 6))
    toks = list(range(100, 122))
    m.admit_with_prefix("a", toks)
    m.register_full_pages("a", toks, 22)
    wa = list(m.table("a", 1))
    m.release("a")
    assert m.can_admit(toks) == 5
    # window page 3 is taken again by another request: hits that need it (n = 4 and 5) are gone,
    # n = 3 needs window pages 1 and 2 only
    pool = m.pools[1]
    while pool.hash_to_page.get(pool.hash_of[wa[3]]) == wa[3]:
        pool.take()
    hits, pages = m.match_prefix(toks)
    taken = [p for p in range(pool.num_pages) if pool.ref_count[p]]
    for p in taken:
        pool.give_back(p)
    assert hits == 3 and pages[1] == [-1, wa[1], wa[2]] and len(pages[0]) == 3
    # an all-keys page that is gone ends the chain there
    m2 = _manager(pages=12, page=4, groups=(None, 6))
    m2.admit_with_prefix("a", toks)
    m2.register_full_pages("a", toks, 22)
    t2 = list(m2.table("a", 0))
    m2.release("a")
    m2.pools[0].tokens_of[t2[2]] = (0, 0, 0, 0)
    assert m2.can_admit(toks) == 2


def test_random_requests_with_shared_prefixes_over_two_groups():
    """Requests drawn from a few common prefixes come and go in random order on small pools of
    an all-keys and a window group: the books balance after every call, a hit never exceeds what
    was registered, and at the end every page is free."""
    rng = random.Random(5)
    page, window = 4, 10
    m = _manager(pages=40, page=page, groups=(None, window))
    stems = [[rng.randrange(50) for _ in range(rng.randrange(8, 40))] for _ in range(3)]
    live = {}
    hits_seen = 0
    for i in range(400):
        if live and (len(live) >= 4 or rng.random() < 0.4):
            rid = rng.choice(list(live))
            toks, pos = live[rid]
            n = min(len(toks) - pos, rng.choice([1, 2, 5, 9]))
            if m.can_reserve(rid, pos + n, pos, pos + n):
                m.reserve(rid, pos + n, pos, pos + n)
                pos += n
                m.register_full_pages(rid, toks, pos)
                live[rid] = (toks, pos)
            if pos == len(toks) or rng.random() < 0.1:
                m.release(rid)
                del live[rid]
        else:
            toks = rng.choice(stems)[: rng.randrange(5, 40)] + [rng.randrange(50) for _ in range(rng.randrange(1, 9))]
            first = rng.choice([2, 5, 9])
            hits = m.can_admit(toks, first)
            if hits >= 0:
                cached = m.admit_with_prefix(i, toks, first)
                assert cached == hits * page and cached < len(toks)
                hits_seen += hits
                for g, table in enumerate(m.requests[i].tables):
                    lo = m._first_needed_page(g, cached)
                    assert all(p == -1 for p in table[:min(lo, hits)]) and all(p >= 0 for p in table[lo:hits])
                live[i] = (toks, m.requests[i].num_tokens)
                m.register_full_pages(i, toks, cached)
        m.check()
    for rid in list(live):
        m.release(rid)
    m.check()
    assert all(pool.num_free == pool.num_pages for pool in m.pools)
    assert hits_seen > 20


# ------------------------------------------------------------------------------ state slots
def test_state_slots():
    m = _manager(slots=2)
    a, b = m.admit("a"), m.admit("b")
    assert {a.state_slot, b.state_slot} == {0, 1}
    with pytest.raises(OutOfPages):
        m.admit("c")
    m.release("a")
    assert m.admit("c").state_slot == a.state_slot
    m.check()
    pool = SlotPool(1)
    s = pool.take()
    pool.give_back(s)
    with pytest.raises(PageError):
        pool.give_back(s)


def test_reserving_for_several_requests_is_all_or_nothing():
    m = CacheManager([CacheGroup(None, (0,))], 4, 5)
    for r, n in (("a", 7), ("b", 8)):
        m.admit(r)
        m.reserve(r, n)
    assert m.pools[0].num_free == 1
    assert m.can_reserve_all([("a", 8, 7), ("b", 8, 7)])             # no new page
    assert m.can_reserve_all([("a", 12, 7), ("b", 8, 7)])            # one new page: it is there
    assert not m.can_reserve_all([("a", 12, 7), ("b", 12, 7)])       # two are not, though each alone would find one
    assert m.can_reserve("a", 12, 7) and m.can_reserve("b", 12, 7)
    assert m.pools[0].num_free == 1
    m.check()


def test_reserving_for_several_requests_counts_pages_in_the_order_of_the_calls():
    """A window group: b's window has passed two pages that reserve(b) would give back, but a comes
    first and finds no page; the sums over both balance, the calls one after the other fail."""
    m = CacheManager([CacheGroup(8, (0,))], 4, 6)
    m.admit("a")
    m.reserve("a", 8)                        # 2 pages
    m.admit("b")
    m.reserve("b", 16)                       # 4 pages; none is free now
    assert m.pools[0].num_free == 0
    # a query at position 16 with a window of 8 sees positions 9..16: b's pages 0 and 1 have been passed
    wanted = [("a", 9, 8), ("b", 17, 16)]
    assert m.pages_needed("a", 9, 8) == [1] and m._passed_pages("a", 8) == [0]
    assert m.pages_needed("b", 17, 16) == [1] and m._passed_pages("b", 16) == [2]
    assert not m.can_reserve_all(wanted)                 # a, first, would raise OutOfPages
    with pytest.raises(OutOfPages):
        m.reserve("a", 9, first_query=8)
    assert m.can_reserve_all(wanted[::-1])               # b first gives two pages back and takes one, a the other
    m.reserve("b", 17, first_query=16)
    m.reserve("a", 9, first_query=8)
    assert m.pools[0].num_free == 0
    m.check()
