"""The cache manager: pages of keys and values with a block table per request and group.

Replaces the reference's per-sample contiguous caches that grow by copying and
are gathered into a padded batch every step
(/root/reference/src/models/self_attn.cpp:369-389, src/models/cache_batching.cpp:25-81,
src/cuda/ops/self_attn_detail.cuh:951-1008,1109-1142).

Groups: cache slabs whose mixers have the same need (heads, head size, window)
form a group with a page pool and block tables of its own.  A request's block
table in a group lists its pages in token order; all slabs of the group use the
same page ids.  A group with a window gives pages back as soon as every token in
them lies behind the window of the next token; their table entries become -1.

Protocol for one step: `reserve(req, n)` takes the pages that the next n tokens
need in every group (all or nothing), the step writes and reads them,
`commit(req, n)` makes the tokens part of the request and releases pages behind
windows.  `release(req)` gives everything back.  This class holds no device memory.
"""
from __future__ import annotations

from dataclasses import dataclass, field

from ..parts.base import CacheNeed
from .pages import NoFreeSlot, OutOfPages, PagePool, SlotPool

__all__ = ["CacheManager", "RequestCache", "OutOfPages", "NoFreeSlot"]


@dataclass
class RequestCache:
    request_id: object
    slot: int
    num_tokens: int = 0                      # tokens whose keys and values are in the cache
    tables: list[list[int]] = field(default_factory=list)   # per group: page ids, -1 = given back
    live: bool = True
    version: int = 0                         # changes whenever a table changes


def _ceil_div(a: int, b: int) -> int:
    return -(-a // b)


class CacheManager:
    def __init__(self, groups: list[CacheNeed], page_size: int, num_pages, max_requests: int):
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
        self.requests: dict[object, RequestCache] = {}

    # ------------------------------------------------------------------ admission
    def admit(self, request_id) -> RequestCache:
        if request_id in self.requests:
            raise ValueError(f"request {request_id!r} is already live")
        slot = self.slots.take()
        rc = RequestCache(request_id, slot, 0, [[] for _ in self.groups])
        self.requests[request_id] = rc
        return rc

    # ------------------------------------------------------------------ pages for the next tokens
    def pages_needed(self, rc: RequestCache, n_new: int) -> list[int]:
        """Pages each group must still take so that tokens [num_tokens, num_tokens + n_new) have a place."""
        want = _ceil_div(rc.num_tokens + n_new, self.page_size)
        return [max(0, want - len(t)) for t in rc.tables]

    def can_reserve(self, rc: RequestCache, n_new: int, spare=None) -> bool:
        """spare: pages per group already promised to others in the same step."""
        need = self.pages_needed(rc, n_new)
        spare = spare or [0] * len(self.pools)
        return all(n <= pool.free_count - s for n, pool, s in zip(need, self.pools, spare))

    def reserve(self, rc: RequestCache, n_new: int) -> None:
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

    def commit(self, rc: RequestCache, n_new: int) -> None:
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

    def release(self, rc: RequestCache) -> None:
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
    def slot_index(self, rc: RequestCache, group: int, position: int) -> int:
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
