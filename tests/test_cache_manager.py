"""The cache manager's bookkeeping (no GPU): no page lost, held twice or freed twice.

The product's manager is C++ behind ctypes; tests/plain_cache.py is the same protocol in plain Python.  Both go
through the same cases here, and through the same random sequences of operations side by side.
"""
import ctypes
import random

import numpy as np
import pytest

import plain_cache
from easy_gpt.cpp_amd.cache import CacheManager, NoFreeSlot, OutOfPages
from easy_gpt.cpp_amd.parts import CacheNeed
from plain_cache import PagePool, SlotPool

FULL = CacheNeed.keys_and_values(n_kv_heads=2, head_dim=16, window=None)
WIN = CacheNeed.keys_and_values(n_kv_heads=1, head_dim=32, window=10)


def test_page_pool_take_give_back_and_reuse_order():
    p = PagePool(4)
    a = p.take(3)
    assert a == [0, 1, 2] and p.free_count == 1
    p.give_back([1])
    assert p.take(1) == [1]                    # freed last, handed out first
    with pytest.raises(plain_cache.OutOfPages):
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
    with pytest.raises(plain_cache.NoFreeSlot):
        s.take()
    with pytest.raises(RuntimeError):
        s.give_back(99)
    s.check()
    assert b == 1


BOTH = [(CacheManager, OutOfPages, NoFreeSlot),
        (plain_cache.PlainCacheManager, plain_cache.OutOfPages, plain_cache.NoFreeSlot)]


@pytest.mark.parametrize("Manager,OutOfPages,NoFreeSlot", BOTH, ids=["native", "plain"])
def test_reserve_commit_release_full_group(Manager, OutOfPages, NoFreeSlot):
    m = Manager([FULL], page_size=4, num_pages=6, max_requests=2)
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


@pytest.mark.parametrize("Manager,OutOfPages,NoFreeSlot", BOTH, ids=["native", "plain"])
def test_window_group_gives_pages_back_as_the_window_passes(Manager, OutOfPages, NoFreeSlot):
    m = Manager([FULL, WIN], page_size=4, num_pages=[16, 8], max_requests=1)
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


@pytest.mark.parametrize("Manager,OutOfPages,NoFreeSlot", BOTH, ids=["native", "plain"])
def test_reserve_is_all_or_nothing_across_groups(Manager, OutOfPages, NoFreeSlot):
    m = Manager([FULL, WIN], page_size=4, num_pages=[8, 2], max_requests=1)
    r = m.admit("r")
    with pytest.raises(OutOfPages):
        m.reserve(r, 12)                       # group 1 has only 2 pages
    assert r.tables == [[], []] and m.free_pages() == [8, 2]


@pytest.mark.parametrize("seed", range(8))
def test_random_orders_keep_the_invariants_and_both_managers_agree(seed):
    rng = random.Random(seed)
    ps = rng.choice([1, 3, 4, 16])
    pages = [rng.randint(8, 40), rng.randint(6, 20)]
    m = CacheManager([FULL, WIN], page_size=ps, num_pages=pages, max_requests=4)
    ref = plain_cache.PlainCacheManager([FULL, WIN], page_size=ps, num_pages=pages, max_requests=4)
    live, next_id = {}, 0

    def same():
        assert m.free_pages() == ref.free_pages()
        assert [p.high_water for p in m.pools] == [p.high_water for p in ref.pools]
        for rid, (rc, pc) in live.items():
            assert (rc.slot, rc.num_tokens, rc.tables) == (pc.slot, pc.num_tokens, pc.tables), rid

    for _ in range(400):
        op = rng.random()
        if op < 0.2 and len(live) < 4:
            live[next_id] = (m.admit(next_id), ref.admit(next_id))
            next_id += 1
        elif op < 0.85 and live:
            rc, pc = rng.choice(list(live.values()))
            n = rng.choice([1, 1, 1, 2, 5, 17])
            before = [list(t) for t in rc.tables]
            assert m.pages_needed(rc, n) == ref.pages_needed(pc, n)
            assert m.can_reserve(rc, n) == ref.can_reserve(pc, n)
            if m.can_reserve(rc, n):
                m.reserve(rc, n), ref.reserve(pc, n)
                if rng.random() < 0.15:                   # the step fails: what it took goes back
                    m.unreserve_step([rc]), ref.unreserve_step([pc])
                    assert [list(t) for t in rc.tables] == before
                else:
                    m.commit(rc, n), ref.commit(pc, n)
            else:
                with pytest.raises(OutOfPages):
                    m.reserve(rc, n)
                assert [list(t) for t in rc.tables] == before
        elif live:
            rid = rng.choice(list(live))
            rc, pc = live.pop(rid)
            m.release(rc), ref.release(pc)
        m.check(), ref.check()
        same()
    for rc, pc in list(live.values()):
        m.release(rc), ref.release(pc)
    m.check()
    assert m.free_pages() == [p.num_pages for p in m.pools]


def test_a_step_reserves_for_all_its_requests_or_for_none():
    m = CacheManager([FULL, WIN], page_size=4, num_pages=[6, 6], max_requests=3)
    a, b, c = m.admit("a"), m.admit("b"), m.admit("c")
    with pytest.raises(OutOfPages, match="'c'"):
        m.reserve_step([a, b, c], [8, 8, 9])          # 2 + 2 + 3 pages of 6
    assert m.free_pages() == [6, 6] and a.tables == [[], []]
    m.reserve_step([a, b, c], [8, 8, 8])
    assert m.free_pages() == [0, 0]
    m.commit_step([a, b, c], [8, 8, 8])
    assert (a.num_tokens, b.num_tokens, c.num_tokens) == (8, 8, 8)
    with pytest.raises(RuntimeError, match="without reserve"):
        m.commit(a, 1)
    m.check()


@pytest.mark.parametrize("Manager,OutOfPages,NoFreeSlot", BOTH, ids=["native", "plain"])
def test_a_failed_step_gives_back_what_it_reserved(Manager, OutOfPages, NoFreeSlot):
    m = Manager([FULL, WIN], page_size=4, num_pages=[12, 6], max_requests=3)
    a, b = m.admit("a"), m.admit("b")
    snapshot = lambda: ([list(t) for t in a.tables], [list(t) for t in b.tables])
    for rc, n in ((a, 6), (b, 3)):
        m.reserve(rc, n)
        m.commit(rc, n)
    free, tables = m.free_pages(), snapshot()
    m.reserve(a, 9), m.reserve(b, 2)                   # a: two more pages in each group, b: one more
    taken = snapshot()
    assert m.free_pages() == [free[0] - 3, free[1] - 3]
    m.unreserve_step([a, b])                           # the step failed: nothing was committed
    assert m.free_pages() == free and snapshot() == tables
    assert (a.num_tokens, b.num_tokens) == (6, 3)
    m.check()
    m.reserve(a, 9), m.reserve(b, 2)                   # the same pages come again, in the same order
    assert snapshot() == taken
    m.commit(a, 9), m.commit(b, 2)
    after = snapshot()
    m.unreserve_step([a, b])                           # nothing to give back: every page holds committed tokens
    assert snapshot() == after
    m.release(a), m.release(b)
    m.check()
    assert m.free_pages() == [12, 6]


def test_the_library_writes_a_steps_metadata():
    # what the engine uploads: positions, lengths, slots and block tables, for single tokens and for portions
    ps = 4
    m = CacheManager([FULL, WIN], page_size=ps, num_pages=[20, 20], max_requests=3)
    a, b = m.admit("a"), m.admit("b")
    m.reserve(a, 13), m.commit(a, 13), m.reserve(b, 2), m.commit(b, 2)      # a: pages behind its window are gone
    # --- one token each
    m.reserve_step([b, a], [1, 1])
    n, widths = 2, [4, 4]
    small = np.full((7 + 2) * n, -7, dtype=np.int32)
    tab = np.full(sum(n * w for w in widths), -7, dtype=np.int32)
    state = np.full(2 * n, -1, dtype=np.int64)
    handles = (ctypes.c_int32 * n)(b.handle, a.handle)
    cw = (ctypes.c_int32 * 2)(*widths)
    assert m.fill_decode(handles, cw, small.ctypes.data, tab.ctypes.data, state.ctypes.data) is True
    rows = small.reshape(9, n)
    assert list(rows[0]) == [-7, -7]                                           # token ids are the caller's
    assert list(rows[1]) == [2, 13] and list(rows[4]) == [3, 14]               # positions, kv lengths
    assert list(rows[2]) == [0, 1] and list(rows[3]) == [1, 1] and list(rows[6]) == [0, 1]
    assert list(rows[5]) == [b.slot, a.slot]
    assert list(rows[7]) == [m.slot_index(b, 0, 2), m.slot_index(a, 0, 13)]
    assert list(rows[8]) == [m.slot_index(b, 1, 2), m.slot_index(a, 1, 13)]
    t = tab.reshape(2, n, 4)
    for g in range(2):
        for i, rc in enumerate((b, a)):
            want = rc.tables[g] + [-1] * (4 - len(rc.tables[g]))
            assert list(t[g, i]) == want
    assert a.tables[1][0] == -1                                                # a page behind the window
    tab[:] = -7
    assert m.fill_decode(handles, cw, small.ctypes.data, tab.ctypes.data, state.ctypes.data) is False
    assert (tab == -7).all()                                                   # unchanged rows are not rewritten
    m.commit_step([b, a], [1, 1])
    m.reserve_step([b], [2])                                                   # b's table grows: its row is rewritten
    assert m.fill_decode(handles, cw, small.ctypes.data, tab.ctypes.data, state.ctypes.data) is True
    assert list(tab.reshape(2, n, 4)[0, 0]) == b.tables[0] + [-1] * (4 - len(b.tables[0]))
    assert (tab.reshape(2, n, 4)[:, 1] == -7).all()
    # --- portions
    counts, total = [2, 1], 3
    bufs = [np.full(k, -7, dtype=np.int32) for k in (total, n, n, n, n, 2 * total, sum(n * w for w in widths))]
    m.reserve_step([b, a], counts)
    m.fill_step((ctypes.c_int32 * n)(b.handle, a.handle), (ctypes.c_int32 * n)(*counts), cw, [x.ctypes.data for x in bufs])
    positions, q_start, q_len, kv_len, slots_state, slots, tables = bufs
    assert list(positions) == [3, 4, 14] and list(q_start) == [0, 2] and list(q_len) == [2, 1]
    assert list(kv_len) == [5, 15] and list(slots_state) == [b.slot, a.slot]
    assert list(slots[:total]) == [m.slot_index(b, 0, 3), m.slot_index(b, 0, 4), m.slot_index(a, 0, 14)]
    assert list(slots[total:]) == [m.slot_index(b, 1, 3), m.slot_index(b, 1, 4), m.slot_index(a, 1, 14)]
    assert list(tables.reshape(2, n, 4)[1, 1]) == a.tables[1] + [-1] * (4 - len(a.tables[1]))
    m.check()
