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
need in every group (all or nothing; `reserve_step` does it for all requests of a
step at once), the step writes and reads them, `commit(req, n)` makes the tokens
part of the request and releases pages behind windows.  `release(req)` gives
everything back.  This class holds no device memory.

The bookkeeping itself (pools, tables, slots, the invariants) and the packing of a
step's metadata into the engine's pinned buffers are C++ (csrc/host/cache_core.cpp);
this module is its binding.  It mirrors the few numbers that the scheduler reads in
its inner loops (tokens per request, table lengths, free pages), so that planning a
step costs no calls into the library.
"""
from __future__ import annotations

import contextlib
import ctypes

from ..parts.base import CacheNeed


class OutOfPages(RuntimeError):
    """Not enough free pages; nothing was taken."""


class NoFreeSlot(RuntimeError):
    """Every request slot is in use."""


__all__ = ["CacheManager", "RequestCache", "OutOfPages", "NoFreeSlot"]

EGH_NO_SLOT, EGH_BAD_HANDLE, EGH_OUT_OF_PAGES, EGH_BAD_ARGUMENT, EGH_NO_PAGE, EGH_INVARIANT = -1, -2, -3, -4, -5, -6
_I32P = ctypes.POINTER(ctypes.c_int32)
_lib = None


def _library():
    global _lib
    if _lib is None:
        from ..csrc import build

        lib = ctypes.CDLL(build.ensure_host_built())
        if lib.egh_abi_version() != 3:
            raise RuntimeError("the host library has an unexpected ABI version")
        vp, i = ctypes.c_void_p, ctypes.c_int
        sigs = {
            "egh_create": ([i, vp, vp, i, i], vp), "egh_destroy": ([vp], None), "egh_admit": ([vp], i),
            "egh_release": ([vp, i], i), "egh_slot": ([vp, i], i), "egh_num_tokens": ([vp, i], i),
            "egh_version": ([vp, i], i), "egh_table_len": ([vp, i, i], i), "egh_table": ([vp, i, i, vp, i], i),
            "egh_pages_needed": ([vp, i, i, vp], i), "egh_free_pages": ([vp, i], i), "egh_used_pages": ([vp, i], i),
            "egh_num_pages": ([vp, i], i), "egh_high_water": ([vp, i], i), "egh_free_slots": ([vp], i),
            "egh_reserve": ([vp, i, vp, vp, vp], i), "egh_commit": ([vp, i, vp, vp], i), "egh_unreserve": ([vp, i, vp], i),
            "egh_slot_index": ([vp, i, i, i], i), "egh_check": ([vp, vp, i], i),
            "egh_fill_decode": ([vp, i, vp, vp, vp, vp, vp], i),
            "egh_fill_decode_rows": ([vp, i, i, vp, vp, vp, vp, vp], i),
            "egh_fill_step": ([vp, i, vp, vp, vp, vp, vp, vp, vp, vp, vp, vp], i),
        }
        for name, (args, res) in sigs.items():
            fn = getattr(lib, name)
            fn.argtypes, fn.restype = args, res
        _lib = lib
    return _lib


def _ints(values):
    return (ctypes.c_int32 * len(values))(*values)


class RequestCache:
    """A live request's place in the cache.  `num_tokens` (tokens whose keys and values are in the cache) and
    `table_lens` (entries of its block table, per group) mirror the library's state."""

    __slots__ = ("request_id", "handle", "slot", "num_tokens", "table_lens", "live", "_manager")

    def __init__(self, request_id, handle: int, slot: int, n_groups: int, manager):
        self.request_id, self.handle, self.slot = request_id, handle, slot
        self.num_tokens = 0
        self.table_lens = [0] * n_groups
        self.live = True
        self._manager = manager

    @property
    def tables(self) -> list[list[int]]:
        """Per group: page ids in token order, -1 = given back."""
        if not self.live:
            return [[] for _ in self.table_lens]
        lib, core = _library(), self._manager._core
        out = []
        for g in range(len(self.table_lens)):
            n = lib.egh_table_len(core, self.handle, g)
            buf = (ctypes.c_int32 * max(n, 1))()
            lib.egh_table(core, self.handle, g, buf, n)
            out.append(list(buf[:n]))
        return out

    @property
    def version(self) -> int:
        """Changes whenever a table of the request changes."""
        return _library().egh_version(self._manager._core, self.handle) if self.live else -1


class PoolView:
    """A group's page pool as the scheduler sees it; `free_count` and `high_water` are refreshed after every
    call that moves pages."""

    __slots__ = ("num_pages", "free_count", "high_water")

    def __init__(self, num_pages: int):
        self.num_pages = num_pages
        self.free_count = num_pages
        self.high_water = 0

    @property
    def used_count(self) -> int:
        return self.num_pages - self.free_count


class SlotView:
    __slots__ = ("num_slots", "free_count")

    def __init__(self, num_slots: int):
        self.num_slots = self.free_count = num_slots


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
        if any(n < 0 for n in counts):
            raise ValueError("num_pages must be >= 0")
        self._lib = _library()
        windows = [int(g.window) if g.window is not None else 0 for g in self.groups]
        self._core = self._lib.egh_create(len(self.groups), _ints(windows), _ints(counts), self.page_size, int(max_requests))
        if not self._core:
            raise ValueError("the cache manager could not be created from these sizes")
        self.pools = [PoolView(n) for n in counts]
        self.slots = SlotView(int(max_requests))
        self.requests: dict[object, RequestCache] = {}

    def __del__(self):
        core, self._core = getattr(self, "_core", None), None
        if core and _lib is not None:
            _lib.egh_destroy(core)

    def _refresh(self) -> None:
        lib, core = self._lib, self._core
        for g, pool in enumerate(self.pools):
            pool.free_count = lib.egh_free_pages(core, g)
            pool.high_water = lib.egh_high_water(core, g)

    # ------------------------------------------------------------------ admission
    def admit(self, request_id) -> RequestCache:
        if request_id in self.requests:
            raise ValueError(f"request {request_id!r} is already live")
        h = self._lib.egh_admit(self._core)
        if h == EGH_NO_SLOT:
            raise NoFreeSlot(f"all {self.slots.num_slots} request slots are in use")
        if h < 0:
            raise RuntimeError(f"admit failed with code {h}")
        rc = RequestCache(request_id, h, self._lib.egh_slot(self._core, h), len(self.groups), self)
        self.requests[request_id] = rc
        self.slots.free_count -= 1
        return rc

    # ------------------------------------------------------------------ pages for the next tokens
    def pages_needed(self, rc: RequestCache, n_new: int) -> list[int]:
        """Pages each group must still take so that tokens [num_tokens, num_tokens + n_new) have a place."""
        want = -(-(rc.num_tokens + n_new) // self.page_size)
        return [max(0, want - n) for n in rc.table_lens]

    def can_reserve(self, rc: RequestCache, n_new: int, spare=None) -> bool:
        """spare: pages per group already promised to others in the same step."""
        need = self.pages_needed(rc, n_new)
        spare = spare or [0] * len(self.pools)
        return all(n <= pool.free_count - s for n, pool, s in zip(need, self.pools, spare))

    def reserve(self, rc: RequestCache, n_new: int) -> None:
        self.reserve_step([rc], [n_new])

    def reserve_step(self, rcs, counts) -> None:
        """Pages for the next counts[i] tokens of every request of a step: all of them or none."""
        for rc in rcs:
            if not rc.live:
                raise RuntimeError(f"request {rc.request_id!r} was released")
        detail = (ctypes.c_int32 * 4)()
        code = self._lib.egh_reserve(self._core, len(rcs), _ints([rc.handle for rc in rcs]), _ints(list(counts)), detail)
        if code == EGH_OUT_OF_PAGES:
            i, g, need, free = detail[0], detail[1], detail[2], detail[3]
            raise OutOfPages(
                f"request {rcs[i].request_id!r} needs {need} more pages in cache group {g}, "
                f"{free} of {self.pools[g].num_pages} are free"
            )
        if code != 0:
            raise RuntimeError(f"reserve failed with code {code}")
        ps = self.page_size
        for rc, n in zip(rcs, counts):
            want = -(-(rc.num_tokens + n) // ps)
            rc.table_lens = [max(want, have) for have in rc.table_lens]
        self._refresh()

    def unreserve_step(self, rcs) -> None:
        """Gives back what `reserve_step` took for tokens that were not committed (the step failed in between):
        every request keeps the pages of its committed tokens, the pools are as before the reservation."""
        live = [rc for rc in rcs if rc.live]
        code = self._lib.egh_unreserve(self._core, len(live), _ints([rc.handle for rc in live]))
        if code != 0:
            raise RuntimeError(f"unreserve failed with code {code}")
        ps = self.page_size
        for rc in live:
            keep = -(-rc.num_tokens // ps)
            rc.table_lens = [min(keep, have) for have in rc.table_lens]
        self._refresh()

    @contextlib.contextmanager
    def reserved(self, rcs, counts):
        """`with cache.reserved(rcs, counts): run the step`: pages for the step's tokens, committed when the body
        ends and given back when it raises."""
        self.reserve_step(rcs, counts)
        try:
            yield
        except BaseException:
            self.unreserve_step(rcs)
            raise
        self.commit_step(rcs, counts)

    def commit(self, rc: RequestCache, n_new: int) -> None:
        self.commit_step([rc], [n_new])

    def commit_step(self, rcs, counts) -> None:
        code = self._lib.egh_commit(self._core, len(rcs), _ints([rc.handle for rc in rcs]), _ints(list(counts)))
        if code == EGH_NO_PAGE:
            raise RuntimeError("commit without reserve: tokens have no pages")
        if code != 0:
            raise RuntimeError(f"commit failed with code {code}")
        for rc, n in zip(rcs, counts):
            rc.num_tokens += n
        if any(g.window is not None for g in self.groups):
            self._refresh()

    def release(self, rc: RequestCache) -> None:
        if not rc.live:
            raise RuntimeError(f"request {rc.request_id!r} is released twice")
        code = self._lib.egh_release(self._core, rc.handle)
        if code != 0:
            raise RuntimeError(f"release failed with code {code}")
        rc.live = False
        rc.table_lens = [0] * len(self.groups)
        self.slots.free_count += 1
        del self.requests[rc.request_id]
        self._refresh()

    # ------------------------------------------------------------------ queries
    def slot_index(self, rc: RequestCache, group: int, position: int) -> int:
        """page * page_size + offset of the token at `position`."""
        v = self._lib.egh_slot_index(self._core, rc.handle, group, position)
        if v == EGH_NO_PAGE:
            raise RuntimeError("position lies in a page that was given back")
        if v < 0:
            raise RuntimeError(f"slot_index failed with code {v}")
        return v

    def free_pages(self) -> list[int]:
        return [p.free_count for p in self.pools]

    def pages_for_tokens(self, n_tokens: int) -> int:
        return -(-n_tokens // self.page_size)

    def check(self) -> None:
        """Invariants: no page lost, none held twice, tables and pools agree; and the mirrors are true."""
        msg = ctypes.create_string_buffer(200)
        code = self._lib.egh_check(self._core, msg, 200)
        assert code == 0, msg.value.decode()
        for g, pool in enumerate(self.pools):
            assert pool.free_count == self._lib.egh_free_pages(self._core, g), "free page count out of date"
        assert self.slots.free_count == self._lib.egh_free_slots(self._core), "free slot count out of date"
        for rc in self.requests.values():
            assert rc.num_tokens == self._lib.egh_num_tokens(self._core, rc.handle), "token count out of date"
            assert rc.table_lens == [self._lib.egh_table_len(self._core, rc.handle, g) for g in range(len(self.groups))]

    # ------------------------------------------------------------------ a step's metadata, written by the library
    def fill_decode(self, handles, widths, small_ptr: int, tab_ptr: int, row_state_ptr: int, rows: int | None = None) -> bool:
        """One token per request: positions, lengths, slots and (where they changed) block-table rows, written
        into the caller's int32 buffers (layout in csrc/host/cache_core.h), which are laid out for `rows` requests
        (default: as many as there are handles).  True if a table row was rewritten."""
        n = len(handles)
        code = self._lib.egh_fill_decode_rows(self._core, n, n if rows is None else rows, handles, widths, small_ptr,
                                              tab_ptr, row_state_ptr)
        if code == EGH_NO_PAGE:
            raise RuntimeError("a token of this step would be stored in a page that was given back")
        if code < 0:
            raise RuntimeError(f"fill_decode failed with code {code}")
        return code == 1

    def fill_step(self, handles, counts, widths, ptrs) -> None:
        """Any mix of portions: ptrs = addresses of positions, q_start, q_len, kv_len, state_slots, slots, tables."""
        code = self._lib.egh_fill_step(self._core, len(handles), handles, counts, widths, *ptrs)
        if code == EGH_NO_PAGE:
            raise RuntimeError("a token of this step would be stored in a page that was given back")
        if code < 0:
            raise RuntimeError(f"fill_step failed with code {code}")
