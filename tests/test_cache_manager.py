"""The cache manager's bookkeeping (no GPU): no page lost, held twice or freed twice."""
import random

import pytest

from easy_gpt.cpp_amd.cache import CacheManager, NoFreeSlot, OutOfPages, PagePool, SlotPool
from easy_gpt.cpp_amd.parts import CacheNeed

FULL = CacheNeed(n_kv_heads=2, head_dim=16, window=None)
WIN = CacheNeed(n_kv_heads=1, head_dim=32, window=10)


def test_page_pool_take_give_back_and_reuse_order():
    p = PagePool(4)
    a = p.take(3)
    assert a == [0, 1, 2] and p.free_count == 1
    p.give_back([1])
    assert p.take(1) == [1]                    # freed last, handed out first
    with pytest.raises(OutOfPages):
        p.take(2)
    assert p.free_count == 1                   # nothing was taken by the failed call
    p.give_back([0, 2])
    with pytest.raises(RuntimeError, match="not in use"):
        p.give_back([0])                       # freed twice
    with pytest.raises(RuntimeError):
        p.give_back([1, 1])
    p.check()
    assert p.high_water == 3


def test_slot_pool_is_a_stack():
    s = SlotPool(3)
    a, b = s.take(), s.take()
    s.give_back(a)
    assert s.take() == a
    s.take()
    with pytest.raises(NoFreeSlot):
        s.take()
    with pytest.raises(RuntimeError):
        s.give_back(99)
    s.check()
    assert b == 1


def test_reserve_commit_release_full_group():
    m = CacheManager([FULL], page_size=4, num_pages=6, max_requests=2)
    a = m.admit("a")
    assert m.pages_needed(a, 9) == [3]
    m.reserve(a, 9)
    assert a.tables[0] == [0, 1, 2] and a.num_tokens == 0
    m.commit(a, 9)
    assert a.num_tokens == 9 and m.pages_needed(a, 3) == [0] and m.pages_needed(a, 4) == [1]
    assert m.slot_index(a, 0, 0) == 0 and m.slot_index(a, 0, 5) == 1 * 4 + 1 and m.slot_index(a, 0, 8) == 8
    b = m.admit("b")
    with pytest.raises(OutOfPages):
        m.reserve(b, 13)                       # needs 4, only 3 free
    assert b.tables[0] == [] and m.free_pages() == [3]
    m.reserve(b, 12)
    m.commit(b, 12)
    with pytest.raises(OutOfPages):
        m.reserve(a, 4)
    m.release(b)
    assert m.free_pages() == [3]
    m.reserve(a, 4)
    assert a.tables[0][-1] == 5                # b's last page, used again first
    with pytest.raises(RuntimeError, match="twice"):
        m.release(b)
    with pytest.raises(NoFreeSlot):
        m.admit("c"), m.admit("d")
    m.check()


def test_window_group_gives_pages_back_as_the_window_passes():
    m = CacheManager([FULL, WIN], page_size=4, num_pages=[16, 8], max_requests=1)
    r = m.admit("r")
    for n in [3, 6, 1, 1, 7, 2, 12, 1, 1, 1]:
        m.reserve(r, n)
        m.commit(r, n)
        m.check()
        first_needed = max(0, r.num_tokens - WIN.window + 1)
        table = r.tables[1]
        for i, p in enumerate(table):
            wholly_behind = (i + 1) * 4 <= first_needed
            assert (p == -1) == wholly_behind
        assert all(p >= 0 for p in r.tables[0])            # the full group keeps everything
    assert r.num_tokens == 35
    assert sum(p >= 0 for p in r.tables[1]) <= 4
    with pytest.raises(RuntimeError, match="given back"):
        m.slot_index(r, 1, 0)
    m.release(r)
    assert m.free_pages() == [16, 8]


def test_reserve_is_all_or_nothing_across_groups():
    m = CacheManager([FULL, WIN], page_size=4, num_pages=[8, 2], max_requests=1)
    r = m.admit("r")
    with pytest.raises(OutOfPages):
        m.reserve(r, 12)                       # group 1 has only 2 pages
    assert r.tables == [[], []] and m.free_pages() == [8, 2]


@pytest.mark.parametrize("seed", range(8))
def test_random_orders_keep_the_invariants(seed):
    rng = random.Random(seed)
    ps = rng.choice([1, 3, 4, 16])
    m = CacheManager([FULL, WIN], page_size=ps, num_pages=[rng.randint(8, 40), rng.randint(6, 20)], max_requests=4)
    live, next_id = {}, 0
    for _ in range(400):
        op = rng.random()
        if op < 0.2 and len(live) < 4:
            live[next_id] = m.admit(next_id)
            next_id += 1
        elif op < 0.85 and live:
            rc = rng.choice(list(live.values()))
            n = rng.choice([1, 1, 1, 2, 5, 17])
            before = [list(t) for t in rc.tables]
            if m.can_reserve(rc, n):
                m.reserve(rc, n)
                m.commit(rc, n)
            else:
                with pytest.raises(OutOfPages):
                    m.reserve(rc, n)
                assert [list(t) for t in rc.tables] == before
        elif live:
            rid = rng.choice(list(live))
            m.release(live.pop(rid))
        m.check()
    for rc in list(live.values()):
        m.release(rc)
    m.check()
    assert m.free_pages() == [p.num_pages for p in m.pools]
