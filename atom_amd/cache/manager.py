"""The cache manager: pure bookkeeping of pages and state slots, no tensors.

Keys and values live in pages of ``page_size`` tokens.  Layers with the same needs form
a *group*; each group has a pool of pages of its own and, per request, a block table
that lists the request's pages in order of position.  A group with a window keeps only
the pages a later query can still see: once every token of a page is further back than
the window, the page goes back to the pool and its place in the table becomes -1.
Beside the pages there are slots for per-request state of fixed size: a request holds
one slot from its first step to its end, whether the model has such state or not.

What is given back when: all pages and the slot when a request ends or is preempted
(``close``); a window group's pages as the window passes them (``commit``).

Free pages are handed out lowest id first (atom/model_engine/block_pool.py:153-173 hands
out never-used blocks lowest id first), which makes reuse deterministic.  The block math
follows atom/model_engine/block_manager.py:1109-1133 (``can_append``/``may_append``) and
:447-470 (``allocate``).
"""

from __future__ import annotations

import heapq
from dataclasses import dataclass

import numpy as np


class OutOfPages(RuntimeError):
    pass


class OutOfSlots(RuntimeError):
    pass


@dataclass(frozen=True)
class GroupSpec:
    page_size: int
    num_pages: int
    window: int | None = None  # None: every key is kept


class PagePool:
    """Free pages of one group, lowest id first."""

    def __init__(self, num_pages: int):
        self.num_pages = num_pages
        self._free = list(range(num_pages))
        heapq.heapify(self._free)
        self._held = [False] * num_pages

    @property
    def num_free(self) -> int:
        return len(self._free)

    def take(self) -> int:
        if not self._free:
            raise OutOfPages("no free page")
        page = heapq.heappop(self._free)
        assert not self._held[page], f"page {page} was free and held at once"
        self._held[page] = True
        return page

    def give(self, page: int) -> None:
        if not (0 <= page < self.num_pages) or not self._held[page]:
            raise AssertionError(f"page {page} is given back but is not held")
        self._held[page] = False
        heapq.heappush(self._free, page)

    def is_held(self, page: int) -> bool:
        return self._held[page]


class StateSlots:
    """Slots for per-request state of fixed size, lowest free slot first."""

    def __init__(self, num_slots: int):
        self.num_slots = num_slots
        self._free = list(range(num_slots))
        heapq.heapify(self._free)
        self._held = [False] * num_slots

    @property
    def num_free(self) -> int:
        return len(self._free)

    def claim(self) -> int:
        if not self._free:
            raise OutOfSlots("no free state slot")
        slot = heapq.heappop(self._free)
        self._held[slot] = True
        return slot

    def release(self, slot: int) -> None:
        if not (0 <= slot < self.num_slots) or not self._held[slot]:
            raise AssertionError(f"state slot {slot} is released but is not held")
        self._held[slot] = False
        heapq.heappush(self._free, slot)


@dataclass
class _Request:
    tables: list[list[int]]   # per group: page id per page index, -1 where none is held
    slot: int
    fresh: bool = True        # no step has run for it yet
    serial: int = 0           # unique per ``open``: a request id that is opened again gets a new one


class CacheManager:
    def __init__(self, groups: list[GroupSpec], num_state_slots: int):
        if not groups:
            groups = []
        for g in groups:
            if g.page_size <= 0 or g.num_pages < 0:
                raise ValueError(f"bad group {g}")
            if g.window is not None and g.window <= 0:
                raise ValueError("a window must be positive")
        self.groups = list(groups)
        self.pools = [PagePool(g.num_pages) for g in groups]
        self.slots = StateSlots(num_state_slots)
        self._requests: dict[object, _Request] = {}
        self._opened = 0

    # ------------------------------------------------------------------ requests

    def __contains__(self, req_id) -> bool:
        return req_id in self._requests

    def live_requests(self) -> list:
        return list(self._requests)

    def can_open(self) -> bool:
        return self.slots.num_free > 0

    def open(self, req_id) -> int:
        """Registers a request and claims its state slot."""
        if req_id in self._requests:
            raise KeyError(f"request {req_id!r} is already open")
        slot = self.slots.claim()
        self._opened += 1
        self._requests[req_id] = _Request([[] for _ in self.groups], slot, serial=self._opened)
        return slot

    def close(self, req_id) -> None:
        """Gives back every page (last first) and the state slot."""
        req = self._requests.pop(req_id)
        for pool, table in zip(self.pools, req.tables):
            for page in reversed(table):
                if page >= 0:
                    pool.give(page)
        self.slots.release(req.slot)

    def state_slot(self, req_id) -> int:
        return self._requests[req_id].slot

    def serial(self, req_id) -> int:
        """A number no other opening of any request has: tells a re-opened request from its earlier life."""
        return self._requests[req_id].serial

    def is_fresh(self, req_id) -> bool:
        return self._requests[req_id].fresh

    # ------------------------------------------------------------------ pages

    def _first_page_needed(self, group: int, cached: int) -> int:
        """Index of the first page a query at position >= ``cached`` can still see."""
        g = self.groups[group]
        if g.window is None:
            return 0
        return max(0, cached - g.window + 1) // g.page_size

    def _end_for(self, group: int, upto: int, reserve: int | None) -> int:
        # groups that keep every key may reserve beyond this step (the whole prompt at
        # admission); a window group holds only what the step needs
        if reserve is not None and self.groups[group].window is None:
            return max(upto, reserve)
        return upto

    def pages_missing(self, req_id, cached: int, upto: int, reserve: int | None = None) -> list[int]:
        """Per group, how many new pages a step over positions [cached, upto) needs.  An
        unknown request counts from nothing."""
        req = self._requests.get(req_id)
        out = []
        for gi, g in enumerate(self.groups):
            end = self._end_for(gi, upto, reserve)
            if end <= 0:
                out.append(0)
                continue
            last = (end - 1) // g.page_size
            table = req.tables[gi] if req else []
            if g.window is None:
                # nothing is given back before the request ends: the table has no gaps
                out.append(max(0, last + 1 - len(table)))
                continue
            first = self._first_page_needed(gi, cached)
            need = 0
            for idx in range(first, last + 1):
                if idx >= len(table) or table[idx] < 0:
                    need += 1
            out.append(need)
        return out

    def can_cover(self, req_id, cached: int, upto: int, reserve: int | None = None) -> bool:
        return all(need <= pool.num_free
                   for need, pool in zip(self.pages_missing(req_id, cached, upto, reserve), self.pools))

    def cover(self, req_id, cached: int, upto: int, reserve: int | None = None) -> None:
        """Makes sure positions [cached, upto), and whatever earlier positions their queries
        still see, have pages.  All or nothing: raises ``OutOfPages`` before taking any."""
        if not self.can_cover(req_id, cached, upto, reserve):
            raise OutOfPages(f"request {req_id!r}: pages for positions [{cached}, {upto}) are not available")
        req = self._requests[req_id]
        for gi, g in enumerate(self.groups):
            end = self._end_for(gi, upto, reserve)
            if end <= 0:
                continue
            last = (end - 1) // g.page_size
            table = req.tables[gi]
            if g.window is None:
                while len(table) <= last:
                    table.append(self.pools[gi].take())
                continue
            first = self._first_page_needed(gi, cached)
            while len(table) <= last:
                table.append(-1)
            for idx in range(first, last + 1):
                if table[idx] < 0:
                    if idx * g.page_size + g.page_size <= cached:
                        # a page wholly behind the cached tokens can only be missing because the
                        # window passed it; a query that needs it again would read nothing
                        raise AssertionError(f"request {req_id!r}: page {idx} was given back and is needed again")
                    table[idx] = self.pools[gi].take()

    def commit(self, req_id, cached_after: int) -> None:
        """After a step: ``cached_after`` tokens are in the cache.  Pages of window groups that
        no later query can see are given back."""
        req = self._requests[req_id]
        req.fresh = False
        for gi, g in enumerate(self.groups):
            if g.window is None:
                continue
            first = self._first_page_needed(gi, cached_after)
            table = req.tables[gi]
            for idx in range(min(first, len(table))):
                if table[idx] >= 0:
                    self.pools[gi].give(table[idx])
                    table[idx] = -1

    def block_table(self, req_id, group: int) -> list[int]:
        return self._requests[req_id].tables[group]

    def slot_mapping(self, req_id, group: int, start: int, count: int) -> np.ndarray:
        """Cache slot (page * page_size + offset) of positions start .. start + count - 1."""
        g = self.groups[group]
        table = np.asarray(self._requests[req_id].tables[group], dtype=np.int64)
        pos = np.arange(start, start + count, dtype=np.int64)
        pages = table[pos // g.page_size]
        if (pages < 0).any():
            raise AssertionError(f"request {req_id!r}: a position in [{start}, {start + count}) has no page")
        return (pages * g.page_size + pos % g.page_size).astype(np.int32)

    def num_free_pages(self, group: int = 0) -> int:
        return self.pools[group].num_free

    # ------------------------------------------------------------------ checks

    def check(self) -> None:
        """No page lost, none held twice, none both free and held; same for slots."""
        for gi, (g, pool) in enumerate(zip(self.groups, self.pools)):
            held = []
            for req in self._requests.values():
                held.extend(p for p in req.tables[gi] if p >= 0)
            assert len(held) == len(set(held)), f"group {gi}: a page is held twice"
            free = list(pool._free)
            assert len(free) == len(set(free)), f"group {gi}: a page is free twice"
            assert not (set(free) & set(held)), f"group {gi}: a page is free and held"
            assert len(free) + len(held) == g.num_pages, f"group {gi}: {g.num_pages - len(free) - len(held)} page(s) lost"
            for p in held:
                assert pool.is_held(p)
        slots = [r.slot for r in self._requests.values()]
        assert len(slots) == len(set(slots)), "a state slot is held twice"
        assert len(slots) + self.slots.num_free == self.slots.num_slots, "a state slot is lost"
