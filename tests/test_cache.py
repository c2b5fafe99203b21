"""The cache manager on the CPU: no page is lost, held twice or freed twice, under random orders of
requests; windows give pages back; state slots."""
import random

import pytest
import torch

from ginfer_amd.cache import CacheManager, PagePool, SlotPool, OutOfPages
from ginfer_amd.parts import KVCacheSpec, StateSpec

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
    assert m.group_of == {0: (0, 0), 3: (0, 1), 1: (1, 0), 5: (1, 1)} and m.state_entries == [4]
    assert m.bytes_per_page(2) == 4 * 2 * 2 * 8 * 16 * 2


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
    assert m.table("b", 0) == [4, 5, 0, 1, 2]    # the pages of "a" are used again, after those that were free
    with pytest.raises(ValueError, match="already"):
        m.admit("b")
    m.admit("c")
    with pytest.raises(OutOfPages, match="state slot"):
        m.admit("d")


def test_window_gives_pages_back():
    m = CacheManager([FULL, WIN], page_size=8, num_pages=8, max_requests=1)
    m.admit("a")
    m.append("a", 30)
    m.commit("a")
    assert m.table("a", 1) == [0, 1, 2, 3]
    # the next token sits at 30 and sees positions 11..30: block 0 (positions 0..7) is behind the window
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
