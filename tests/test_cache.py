"""The cache manager on the CPU: no page is lost, held twice or freed twice, under random orders of
requests; windows give pages back; state slots."""
import random

import pytest
import torch

from ginfer_amd.cache import CacheManager, PagePool, SlotPool, OutOfPages
from ginfer_amd.parts import KVCacheSpec, PagedSpec, StateSpec

FULL = KVCacheSpec(2, 16, None)
WIN = KVCacheSpec(2, 16, 20)


def test_page_pool():
    p = PagePool(4)
    a = p.take(3)
    assert a == [0, 1, 2] and p.num_free == 1
    with pytest.raises(OutOfPages):
        p.take(2)
    assert p.num_free == 1                       # a failed take takes nothing
    p.give_back([1])
    with pytest.raises(ValueError, match="not held"):
        p.give_back([1])                         # freed twice
    with pytest.raises(ValueError, match="not of this pool"):
        p.give_back([9])
    assert p.take(2) == [3, 1]                   # first in, first out: a freed page waits its turn
    assert sorted(p.held()) == [0, 1, 2, 3]


def test_page_pool_with_several_holders():
    p = PagePool(3)
    assert p.take(2) == [0, 1]
    p.share(0)
    assert p.holders(0) == 2
    p.give_back([0])
    assert p.holders(0) == 1 and p.num_free == 1          # still held by the other
    p.give_back([0, 1])
    assert p.num_free == 3
    p.share(0)                                            # out of the free queue again, with what it held
    assert p.holders(0) == 1 and p.num_free == 2 and p.take(2) == [2, 1]
    with pytest.raises(ValueError, match="not held"):
        p.give_back([2, 2])


def test_slot_pool():
    s = SlotPool(2)
    assert (s.take(), s.take()) == (0, 1)
    with pytest.raises(OutOfPages):
        s.take()
    s.give_back(0)
    with pytest.raises(ValueError):
        s.give_back(0)
    assert s.take() == 0


def test_groups_by_need():
    m = CacheManager([FULL, WIN, None, FULL, StateSpec((8,), torch.float32), WIN], page_size=8, num_pages=10, max_requests=3)
    assert [(g.spec, g.entries) for g in m.groups] == [(FULL, [0, 3]), (WIN, [1, 5])]
    assert m.group_of == {(0, 0): (0, 0), (3, 0): (0, 1), (1, 0): (1, 0), (5, 0): (1, 1)} and m.state_units == [(4, 0)]
    assert m.pool_bytes(2) == 10 * 4 * 2 * 2 * 8 * 16 * 2


def test_an_entry_may_keep_several_caches_and_pages_of_any_width():
    """A schedule entry's cache may be a list (pages and a state slot side by side); values may be narrower than keys;
    a paged cache may hold any named per-token tensors.  Each distinct paged spec is a group with a pool of its own."""
    narrow = KVCacheSpec(2, 16, None, value_dim=8)
    latent = PagedSpec((("c", 24), ("r", 4)), window=16)
    state = StateSpec((5,), torch.float32)
    m = CacheManager([[narrow, state], FULL, None, [latent, narrow], state], page_size=8, num_pages=[6, 7, 5], max_requests=2)
    assert [(g.spec, g.units) for g in m.groups] == [(narrow, [(0, 0), (3, 1)]), (FULL, [(1, 0)]), (latent, [(3, 0)])]
    assert m.state_units == [(0, 1), (4, 0)]
    # bytes: narrow 2 caches x (2*16 + 2*8) a token, full 1 x 2*2*16, latent 1 x 28; pages of 8 tokens, 2-byte elements
    assert m.pool_bytes(2) == (6 * 2 * 48 + 7 * 64 + 5 * 28) * 8 * 2
    assert CacheManager.state_bytes(m.cache_specs, 2) == 2 * 3 * 5 * 4
    assert not CacheManager.supports_prefix_caching(m.cache_specs)
    counts = CacheManager.plan_pages(m.cache_specs, 8, 2, 10 ** 6, 2, 32, 64)
    assert counts[2] == CacheManager.window_pages(16, 8, 2, 32, 64) and counts[0] == counts[1] > 0
    # a request takes pages in every group alike and gives them all back
    m.admit("a")
    m.append("a", 20)
    m.commit("a")
    assert [len([p for p in m.table("a", gi) if p >= 0]) for gi in range(3)] == [3, 3, 3]
    m.append("a", 20)
    m.commit("a")
    assert [len([p for p in m.table("a", gi) if p >= 0]) for gi in range(3)] == [5, 5, 2]     # the window keeps positions 25 to 39
    m.check()
    m.release("a")
    m.check()
    assert all(g.pool.num_free == g.pool.num_pages for g in m.groups)


def test_append_commit_release_and_reuse():
    m = CacheManager([FULL], page_size=8, num_pages=6, max_requests=2)
    m.admit("a")
    assert m.append("a", 20) == 0 and m.table("a", 0) == [0, 1, 2] and m.pending("a") == 20
    with pytest.raises(ValueError, match="not committed"):
        m.append("a", 1)
    m.commit("a")
    assert m.length("a") == 20
    assert m.append("a", 4) == 20 and m.table("a", 0) == [0, 1, 2]        # room left in the last page
    m.commit("a")
    assert m.append("a", 1) == 24 and m.table("a", 0) == [0, 1, 2, 3]     # a page's edge
    m.commit("a")
    m.admit("b")
    assert m.free_tokens("b") == 16 and m.can_append("b", 16) and not m.can_append("b", 17)
    with pytest.raises(OutOfPages):
        m.append("b", 17)
    m.check()
    assert m.table("b", 0) == []                 # all or nothing
    m.release("a")
    m.check()
    m.append("b", 40)
    # the pages of "a" are used again, after those that were free; the pages of its end first
    assert m.table("b", 0) == [4, 5, 3, 2, 1]
    with pytest.raises(ValueError, match="already"):
        m.admit("b")
    m.admit("c")
    with pytest.raises(OutOfPages, match="state slot"):
        m.admit("d")


def test_window_gives_pages_back():
    m = CacheManager([FULL, WIN], page_size=8, num_pages=8, max_requests=1)
    m.admit("a")
    m.append("a", 30)
    assert m.table("a", 1) == [0, 1, 2, 3]                  # while the step runs, its first query needs block 0
    m.commit("a")
    # the next token sits at 30 and sees positions 11..30: block 0 (positions 0..7) is behind the window and goes back
    # as soon as the 30 tokens are committed
    assert m.table("a", 1) == [-1, 1, 2, 3] and m.groups[1].pool.num_free == 8 - 3
    m.append("a", 1)
    m.commit("a")
    assert m.table("a", 1) == [-1, 1, 2, 3] and m.table("a", 0) == [0, 1, 2, 3]
    for _ in range(25):
        m.append("a", 1)
        m.commit("a")
        m.check()
    # 56 tokens: the next query at 56 sees 37..56 -> blocks 0..3 are behind
    assert m.table("a", 1)[:4] == [-1, -1, -1, -1] and all(p >= 0 for p in m.table("a", 1)[4:])
    assert m.groups[1].pool.num_free == 8 - 3 and m.groups[0].pool.num_free == 1
    # a long portion keeps what its first query needs
    m.release("a")
    m.admit("b")
    m.append("b", 7)
    m.commit("b")
    m.append("b", 50)      # queries 7..56; query 7 sees 0..7
    assert all(p >= 0 for p in m.table("b", 1))
    m.check()


@pytest.mark.parametrize("seed", range(8))
def test_random_orders_keep_every_page_accounted(seed):
    rng = random.Random(seed)
    specs = [FULL, WIN, None, StateSpec((4,), torch.float32), FULL]
    m = CacheManager(specs, page_size=rng.choice([4, 8, 16]), num_pages=rng.choice([12, 30]), max_requests=4)
    live, lengths, next_id = [], {}, 0
    for _ in range(600):
        op = rng.random()
        if op < 0.2 and m.can_admit():
            m.admit(next_id)
            live.append(next_id)
            lengths[next_id] = 0
            next_id += 1
        elif op < 0.85 and live:
            rid = rng.choice(live)
            n = rng.choice([1, 1, 1, 2, 5, 17, 40])
            ok = m.can_append(rid, n)
            before = [list(m.table(rid, g)) for g in range(len(m.groups))]
            try:
                start = m.append(rid, n)
                assert ok and start == lengths[rid]
                # every new position has a page in every group; every position a query of this portion can
                # still see has one too
                for gi, g in enumerate(m.groups):
                    t = m.table(rid, gi)
                    lo = 0 if g.window is None else max(0, start - g.window + 1)
                    for pos in range(lo, start + n):
                        assert t[pos // m.page_size] >= 0
                if rng.random() < 0.9:
                    m.commit(rid)
                    lengths[rid] += n
                else:                                     # the step failed: nothing is committed
                    m.requests[rid].pending = 0
            except OutOfPages:
                assert not ok
                assert before == [list(m.table(rid, g)) for g in range(len(m.groups))]
        elif live:
            rid = live.pop(rng.randrange(len(live)))
            m.release(rid)
            with pytest.raises(KeyError):
                m.release(rid)
        m.check()
    for rid in live:
        m.release(rid)
    m.check()
    assert all(g.pool.num_free == g.pool.num_pages for g in m.groups) and m.slots.num_free == 4


# ---- shared prefixes

def _run(m, rid, tokens, upto=None):
    """Appends and commits the request's tokens from its length up to `upto`."""
    upto = len(tokens) if upto is None else upto
    n = upto - m.length(rid)
    if n > 0:
        m.append(rid, n)
        m.commit(rid, tokens)


def test_prefix_is_shared_exactly():
    m = CacheManager([FULL], page_size=8, num_pages=8, max_requests=3, prefix_caching=True)
    a = list(range(100, 120))                      # 20 tokens: two full pages and a half
    m.admit("a", a)
    assert m.length("a") == 0
    _run(m, "a", a)
    assert m.table("a", 0) == [0, 1, 2]
    b = a[:16] + [7, 7, 7]
    m.admit("b", b)
    assert m.length("b") == 16 and m.table("b", 0) == [0, 1]
    assert m.prefix_hit_tokens == 0                # a hit counts once the request's first tokens are reserved
    assert m.groups[0].pool.holders(0) == 2 and m.groups[0].pool.holders(2) == 1
    m.check()
    _run(m, "b", b)
    assert m.prefix_hit_tokens == 16
    assert m.table("b", 0) == [0, 1, 3]            # its own page from the first token that differs
    m.release("a", a)
    assert m.groups[0].pool.holders(0) == 1 and m.groups[0].pool.num_free == 5
    # a prompt that ends at a page's edge: its last token is left to run, so the last page is not taken over
    m.admit("c", a[:16])
    assert m.length("c") == 8 and m.table("c", 0) == [0]
    m.release("c", a[:16])
    # tokens that differ inside the first page: nothing is shared, although later pages would match
    d = [1] + a[1:]
    m.admit("d", d)
    assert m.length("d") == 0
    m.release("d")
    m.release("b", b)
    m.check()
    assert m.groups[0].pool.num_free == 8
    # everything is free, and still remembered: the same prompt finds its pages again
    m.admit("e", a)
    assert m.length("e") == 16 and m.table("e", 0) == [0, 1]
    m.check()


def test_a_page_taken_for_something_else_is_forgotten_with_what_follows_it():
    m = CacheManager([FULL], page_size=4, num_pages=4, max_requests=2, prefix_caching=True)
    a = [1, 2, 3, 4, 5, 6, 7, 8, 9]
    m.admit("a", a)
    _run(m, "a", a)                                # pages 0, 1 full, 2 begun
    m.release("a", a)                              # free queue: 3, then a's pages from its end: 2, 1, 0
    x = [9] * 13
    m.admit("x", x)
    _run(m, "x", x)                                # takes all four pages: a's are forgotten
    m.release("x")                                 # without tokens: nothing of x is remembered
    m.admit("b", a)
    assert m.length("b") == 0
    _run(m, "b", a, upto=4)                        # the first block again, under a new number
    m.admit("c", a)
    assert m.length("c") == 4                      # the second block of "a" is not found behind the new first one
    m.check()


def test_without_tokens_nothing_is_shared():
    m = CacheManager([FULL], page_size=4, num_pages=6, max_requests=2, prefix_caching=True)
    a = list(range(9))
    m.admit("a")
    m.append("a", 9)
    m.commit("a")
    m.release("a")
    m.admit("b", a)
    assert m.length("b") == 0
    with pytest.raises(ValueError, match="window or with per-request state"):
        CacheManager([FULL, WIN], page_size=4, num_pages=6, max_requests=2, prefix_caching=True)
    with pytest.raises(ValueError, match="window or with per-request state"):
        CacheManager([FULL, StateSpec((4,), torch.float32)], page_size=4, num_pages=6, max_requests=2, prefix_caching=True)
    assert not CacheManager.supports_prefix_caching([None]) and CacheManager.supports_prefix_caching([FULL, None])


@pytest.mark.parametrize("seed", range(8))
def test_random_orders_with_shared_prefixes(seed):
    """Requests whose token lists share beginnings come and go in random order.  A shadow of what every page holds
    (the whole sequence up to the page's end, as the request that wrote it knew it) shows that a page taken over
    holds exactly the newcomer's own beginning."""
    rng = random.Random(100 + seed)
    ps = rng.choice([2, 4, 8])
    specs = [FULL, None, KVCacheSpec(1, 32, None)]
    m = CacheManager(specs, page_size=ps, num_pages=rng.choice([10, 24]), max_requests=4, prefix_caching=True)
    stems = [[rng.randrange(3) for _ in range(40)] for _ in range(3)]
    shadow = [dict() for _ in m.groups]
    live, tokens, next_id, hits = [], {}, 0, 0
    found = {}                # what a request found in the cache counts as a hit once its first tokens are reserved
    for _ in range(800):
        op = rng.random()
        if op < 0.25 and m.can_admit():
            stem = rng.choice(stems)
            cut = rng.randrange(1, 40)
            toks = stem[:cut] + [rng.randrange(3) for _ in range(rng.randrange(0, 12))]
            m.admit(next_id, toks)
            got = m.length(next_id)
            assert got % ps == 0 and got <= len(toks) - 1
            for gi in range(len(m.groups)):
                for i, page in enumerate(m.table(next_id, gi)):
                    assert shadow[gi][page] == toks[:(i + 1) * ps]
            found[next_id] = got
            live.append(next_id)
            tokens[next_id] = toks
            next_id += 1
        elif op < 0.8 and live:
            rid = rng.choice(live)
            toks = tokens[rid]
            start = m.length(rid)
            n = min(rng.choice([1, 1, 2, 3, 7, 20]), len(toks) - start)
            if n == 0:                                   # decoding: a new token becomes known
                toks.append(rng.randrange(3))
                n = 1
            try:
                m.append(rid, n)
            except OutOfPages:
                m.check()
                continue
            hits += found.pop(rid, 0)
            assert hits == m.prefix_hit_tokens
            for gi in range(len(m.groups)):
                t = m.table(rid, gi)
                for blk in range(start // ps, (start + n - 1) // ps + 1):
                    shadow[gi][t[blk]] = toks[:min(start + n, (blk + 1) * ps)]
            m.commit(rid, toks if rng.random() < 0.8 else None)
        elif live:
            rid = live.pop(rng.randrange(len(live)))
            m.release(rid, tokens[rid] if rng.random() < 0.8 else None)
        m.check()
    for rid in live:
        m.release(rid, tokens[rid])
    m.check()
    assert all(g.pool.num_free == g.pool.num_pages for g in m.groups) and m.slots.num_free == 4
    assert hits > 0 and hits == m.prefix_hit_tokens


# ---- how a pool is shared out among groups

def test_a_group_with_a_window_gets_what_a_window_can_hold_and_the_rest_goes_to_all_keys():
    specs = [FULL, WIN, FULL, WIN, None]
    ps, esize, requests, step, longest = 16, 2, 8, 256, 4096
    page_full = 2 * 2 * FULL.num_kv_heads * ps * FULL.head_dim * esize       # two entries, keys and values
    page_win = 2 * 2 * WIN.num_kv_heads * ps * WIN.head_dim * esize
    pool = 64 << 20
    counts = CacheManager.plan_pages(specs, ps, esize, pool, requests, step, longest)
    w = CacheManager.window_pages(WIN.window, ps, requests, step, longest)
    assert w == requests * ((WIN.window - 1) // ps + 3) + step // ps
    assert counts == [(pool - w * page_win) // page_full, w]
    assert counts[0] * page_full > 0.9 * pool                 # nearly all of the pool keeps all keys
    m = CacheManager(specs, ps, counts, requests)
    assert [g.pool.num_pages for g in m.groups] == counts and m.pool_bytes(esize) <= pool
    # a window as long as the longest request is worth no more than all keys
    assert CacheManager.window_pages(10 ** 6, ps, requests, step, longest) == requests * (longest // ps)
    # windows only: each gets what it can hold; too little memory: refused
    assert CacheManager.plan_pages([WIN, WIN], ps, esize, pool, requests, step, longest) == [w]
    with pytest.raises(RuntimeError, match="no memory left"):
        CacheManager.plan_pages(specs, ps, esize, w * page_win + page_full - 1, requests, step, longest)
    with pytest.raises(ValueError, match="page counts"):
        CacheManager(specs, ps, [4], requests)


def test_every_step_fits_the_pages_planned_for_a_window():
    """Whatever portions the requests of a step run, a group with a window never holds more pages than were planned."""
    import random
    ps, requests, step, longest = 8, 4, 40, 400
    win = KVCacheSpec(1, 16, 20)
    pages = CacheManager.window_pages(win.window, ps, requests, step, longest)
    m = CacheManager([win], ps, pages, requests)
    rng = random.Random(3)
    for r in range(requests):
        m.admit(r)
    for _ in range(300):
        budget = step
        for r in rng.sample(range(requests), requests):
            n = min(rng.choice([1, 1, 2, 7, 19, 40]), budget, longest - m.length(r))
            if n > 0:
                m.append(r, n)            # never raises OutOfPages
                budget -= n
        for r in range(requests):
            if m.pending(r):
                m.commit(r)
            if m.length(r) >= longest:
                m.release(r)
                m.admit(r)
        m.check()
