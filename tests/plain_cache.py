"""A plain cache manager in Python: the oracle that the native one (easy_gpt.cpp_amd/cache/manager.py over
csrc/host/cache_core.cpp) is compared with, operation by operation, in tests/test_cache_manager.py.  Same
protocol: reserve (all or nothing), commit (window groups give pages back), release; pages freed last are
handed out first.  Shares no code with the product.
"""
from __future__ import annotations

from dataclasses import dataclass, field


class OutOfPages(RuntimeError):
    pass


class NoFreeSlot(RuntimeError):
    pass

class PagePool:
    """Page ids 0..num_pages-1.  Pages freed last are handed out first, so that reuse
    happens early and a kernel that reads stale contents is caught by the tests."""

    def __init__(self, num_pages: int):
        if num_pages < 0:
            raise ValueError("num_pages must be >= 0")
        self.num_pages = int(num_pages)
        self._free = list(range(self.num_pages - 1, -1, -1))  # pop() gives 0 first
        self._in_use: set[int] = set()
        self.high_water = 0

    @property
    def free_count(self) -> int:
        return len(self._free)

    @property
    def used_count(self) -> int:
        return len(self._in_use)

    def take(self, n: int) -> list[int]:
        if n < 0:
            raise ValueError("cannot take a negative number of pages")
        if n > len(self._free):
            raise OutOfPages(f"{n} pages wanted, {len(self._free)} of {self.num_pages} free")
        pages = [self._free.pop() for _ in range(n)]
        self._in_use.update(pages)
        self.high_water = max(self.high_water, len(self._in_use))
        return pages

    def give_back(self, pages) -> None:
        pages = list(pages)
        for p in pages:
            if p not in self._in_use:
                raise RuntimeError(f"page {p} is given back but not in use (freed twice or never taken)")
        if len(set(pages)) != len(pages):
            raise RuntimeError(f"pages given back twice in one call: {pages}")
        for p in pages:
            self._in_use.remove(p)
            self._free.append(p)

    def check(self) -> None:
        assert len(self._free) + len(self._in_use) == self.num_pages, "a page was lost"
        assert len(set(self._free)) == len(self._free), "a page is on the free list twice"
        assert not (set(self._free) & self._in_use), "a page is both free and in use"


class SlotPool:
    """Slots 0..n-1 for per-request records of fixed size; a stack, as the reference's free
    slot list (/root/reference/src/continuous_batch_server.cpp:44-47,246)."""

    def __init__(self, num_slots: int):
        self.num_slots = int(num_slots)
        self._free = list(range(self.num_slots - 1, -1, -1))
        self._in_use: set[int] = set()

    @property
    def free_count(self) -> int:
        return len(self._free)

    def take(self) -> int:
        if not self._free:
            raise NoFreeSlot(f"all {self.num_slots} request slots are in use")
        s = self._free.pop()
        self._in_use.add(s)
        return s

    def give_back(self, slot: int) -> None:
        if slot not in self._in_use:
            raise RuntimeError(f"slot {slot} is given back but not in use")
        self._in_use.remove(slot)
        self._free.append(slot)

    def check(self) -> None:
        assert len(self._free) + len(self._in_use) == self.num_slots
        assert not (set(self._free) & self._in_use)


@dataclass
class PlainRequestCache:
    request_id: object
    slot: int
    num_tokens: int = 0
    tables: list = field(default_factory=list)
    live: bool = True
    version: int = 0


def _ceil_div(a: int, b: int) -> int:
    return -(-a // b)


class PlainCacheManager:
    """windows: one entry per group, None = the group keeps every key."""

    def __init__(self, groups, page_size: int, num_pages, max_requests: int):
        """groups: one CacheNeed per group.  num_pages: an int (every group gets that many)
        or a list with one count per group."""
        if page_size < 1:
            raise ValueError("page_size must be >= 1")
        self.groups = list(groups)
        self.page_size = int(page_size)
        counts = [num_pages] * len(self.groups) if isinstance(num_pages, int) else list(num_pages)
        if len(counts) != len(self.groups):
            raise ValueError("one page count per group is needed")
        self.pools = [PagePool(n) for n in counts]
        self.slots = SlotPool(max_requests)
        self.requests: dict[object, PlainRequestCache] = {}

    # ------------------------------------------------------------------ admission
    def admit(self, request_id) -> PlainRequestCache:
        if request_id in self.requests:
            raise ValueError(f"request {request_id!r} is already live")
        slot = self.slots.take()
        rc = PlainRequestCache(request_id, slot, 0, [[] for _ in self.groups])
        self.requests[request_id] = rc
        return rc

    # ------------------------------------------------------------------ pages for the next tokens
    def pages_needed(self, rc: PlainRequestCache, n_new: int) -> list[int]:
        """Pages each group must still take so that tokens [num_tokens, num_tokens + n_new) have a place."""
        want = _ceil_div(rc.num_tokens + n_new, self.page_size)
        return [max(0, want - len(t)) for t in rc.tables]

    def can_reserve(self, rc: PlainRequestCache, n_new: int, spare=None) -> bool:
        """spare: pages per group already promised to others in the same step."""
        need = self.pages_needed(rc, n_new)
        spare = spare or [0] * len(self.pools)
        return all(n <= pool.free_count - s for n, pool, s in zip(need, self.pools, spare))

    def reserve(self, rc: PlainRequestCache, n_new: int) -> None:
        if not rc.live:
            raise RuntimeError(f"request {rc.request_id!r} was released")
        need = self.pages_needed(rc, n_new)
        for g, (n, pool) in enumerate(zip(need, self.pools)):
            if n > pool.free_count:
                raise OutOfPages(
                    f"request {rc.request_id!r} needs {n} more pages in cache group {g}, "
                    f"{pool.free_count} of {pool.num_pages} are free"
                )
        for n, pool, table in zip(need, self.pools, rc.tables):
            if n:
                table.extend(pool.take(n))
                rc.version += 1

    def unreserve_step(self, rcs) -> None:
        """Gives back the pages taken for tokens that were not committed, in the reverse of the order of taking."""
        for rc in reversed(list(rcs)):
            keep = _ceil_div(rc.num_tokens, self.page_size)
            for pool, table in reversed(list(zip(self.pools, rc.tables))):
                changed = False
                while len(table) > keep:
                    pool.give_back([table.pop()])
                    changed = True
                if changed:
                    rc.version += 1

    def commit(self, rc: PlainRequestCache, n_new: int) -> None:
        rc.num_tokens += n_new
        if _ceil_div(rc.num_tokens, self.page_size) > min((len(t) for t in rc.tables), default=10**18):
            raise RuntimeError("commit without reserve: tokens have no pages")
        for need, pool, table in zip(self.groups, self.pools, rc.tables):
            if need.window is None:
                continue
            # the next token (position num_tokens) reads keys j > num_tokens - window
            first_needed = rc.num_tokens - need.window + 1
            dead_pages = max(0, first_needed) // self.page_size   # pages wholly below first_needed
            gone = [p for p in table[:dead_pages] if p >= 0]
            if gone:
                pool.give_back(gone)
                for i in range(dead_pages):
                    table[i] = -1
                rc.version += 1

    def release(self, rc: PlainRequestCache) -> None:
        if not rc.live:
            raise RuntimeError(f"request {rc.request_id!r} is released twice")
        for pool, table in zip(self.pools, rc.tables):
            pool.give_back([p for p in table if p >= 0])
            table.clear()
        self.slots.give_back(rc.slot)
        rc.live = False
        rc.version += 1
        del self.requests[rc.request_id]

    # ------------------------------------------------------------------ queries
    def slot_index(self, rc: PlainRequestCache, group: int, position: int) -> int:
        """page * page_size + offset of the token at `position`."""
        page = rc.tables[group][position // self.page_size]
        if page < 0:
            raise RuntimeError("position lies in a page that was given back")
        return page * self.page_size + position % self.page_size

    def free_pages(self) -> list[int]:
        return [p.free_count for p in self.pools]

    def pages_for_tokens(self, n_tokens: int) -> int:
        return _ceil_div(n_tokens, self.page_size)

    def check(self) -> None:
        """Invariants: no page lost, none held twice, tables and pools agree."""
        for g, pool in enumerate(self.pools):
            pool.check()
            held: list[int] = []
            for rc in self.requests.values():
                held.extend(p for p in rc.tables[g] if p >= 0)
            assert len(held) == len(set(held)), f"group {g}: a page is in two block tables"
            assert set(held) == pool._in_use, f"group {g}: block tables and pool disagree"
        self.slots.check()
        slots = [rc.slot for rc in self.requests.values()]
        assert len(slots) == len(set(slots)), "a slot is held by two requests"
        assert set(slots) == self.slots._in_use
