"""A pool of fixed-size pages and a pool of request slots: bookkeeping only, no device memory."""
from __future__ import annotations


class OutOfPages(RuntimeError):
    """Not enough free pages; nothing was taken."""


class NoFreeSlot(RuntimeError):
    """Every request slot is in use."""


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
