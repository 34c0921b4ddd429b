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

Prefix cache (optional, groups that keep every key only): a full page whose tokens have been
run gets a chained content hash (hash of the previous page's hash and its own tokens,
atom/model_engine/block_manager.py:181-187).  A new request takes the longest run of pages whose
hashes match its prompt instead of computing them again, always leaving at least its last token to
be run (block_manager.py:374-379,397).  A hash is published only after the step that filled the page
(:558-626).  Pages are counted by reference; a page with a hash that nobody holds stays findable
until the pool needs it: pages that never had a hash are handed out first, then the least recently
released hashed one, which is then forgotten (atom/model_engine/block_pool.py:153-200).

Free pages are handed out lowest id first (atom/model_engine/block_pool.py:153-173 hands
out never-used blocks lowest id first), which makes reuse deterministic.  The block math
follows atom/model_engine/block_manager.py:1109-1133 (``can_append``/``may_append``) and
:447-470 (``allocate``).
"""

from __future__ import annotations

import heapq
from collections import OrderedDict
from dataclasses import dataclass, field

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
    """Pages of one group, counted by reference.  Free pages without a content hash are handed out
    lowest id first; when none is left, the hashed page released longest ago, whose hash is forgotten."""

    def __init__(self, num_pages: int):
        self.num_pages = num_pages
        self._free = list(range(num_pages))      # no hash, nobody holds them
        heapq.heapify(self._free)
        self._refs = [0] * num_pages
        self._hash: list[int | None] = [None] * num_pages
        self._tokens: list[tuple | None] = [None] * num_pages
        self._by_hash: dict[int, int] = {}
        self._cached: "OrderedDict[int, None]" = OrderedDict()   # hashed, nobody holds them; oldest first
        self.hits = 0
        self.evictions = 0

    @property
    def num_free(self) -> int:
        return len(self._free) + len(self._cached)

    def take(self) -> int:
        if self._free:
            page = heapq.heappop(self._free)
        elif self._cached:
            page, _ = self._cached.popitem(last=False)
            self._forget(page)
            self.evictions += 1
        else:
            raise OutOfPages("no free page")
        assert self._refs[page] == 0, f"page {page} was free and held at once"
        self._refs[page] = 1
        return page

    def give(self, page: int) -> None:
        if not (0 <= page < self.num_pages) or self._refs[page] <= 0:
            raise AssertionError(f"page {page} is given back but is not held")
        self._refs[page] -= 1
        if self._refs[page] == 0:
            if self._hash[page] is not None:
                self._cached[page] = None
            else:
                heapq.heappush(self._free, page)

    def is_held(self, page: int) -> bool:
        return self._refs[page] > 0

    def refs(self, page: int) -> int:
        return self._refs[page]

    # ---- content hashes

    def _forget(self, page: int) -> None:
        h = self._hash[page]
        if h is not None and self._by_hash.get(h) == page:
            del self._by_hash[h]
        self._hash[page] = None
        self._tokens[page] = None

    def publish(self, page: int, content_hash: int, tokens: tuple) -> None:
        """The held page now holds exactly ``tokens`` after the prefix ``content_hash`` chains from.  If
        another page already answers to the hash this one stays anonymous."""
        assert self._refs[page] > 0
        if self._hash[page] is not None or content_hash in self._by_hash:
            return
        self._hash[page] = content_hash
        self._tokens[page] = tokens
        self._by_hash[content_hash] = page

    def find(self, content_hash: int, tokens: tuple) -> int | None:
        """The page that holds this content, or None."""
        page = self._by_hash.get(content_hash)
        if page is None or self._tokens[page] != tokens:
            return None
        return page

    def share(self, page: int) -> None:
        """One more holder of a page found by its hash."""
        if self._refs[page] == 0:
            del self._cached[page]
        self._refs[page] += 1
        self.hits += 1

    def hash_of(self, page: int) -> int | None:
        return self._hash[page]


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
    tokens: list[int] = field(default_factory=list)   # prefix cache: the tokens that are in the cache
    hashes: list[int] = field(default_factory=list)   # prefix cache: chained hash of every full page so far
    unknown_at: int | None = None   # prefix cache: position of a token that ran before the host knew its value


class CacheManager:
    def __init__(self, groups: list[GroupSpec], num_state_slots: int, prefix_caching: bool = False):
        if not groups:
            groups = []
        if prefix_caching and any(g.window is not None for g in groups):
            raise ValueError("the prefix cache needs groups that keep every key")
        if prefix_caching and len({g.page_size for g in groups}) > 1:
            raise ValueError("the prefix cache needs one page size")
        self.prefix_caching = bool(prefix_caching and groups)
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

    # ------------------------------------------------------------------ prefix cache

    @staticmethod
    def _chain(previous: int, tokens: tuple) -> int:
        import xxhash

        h = xxhash.xxh64()
        h.update(previous.to_bytes(8, "little"))
        h.update(np.asarray(tokens, dtype=np.int32).tobytes())
        return h.intdigest()

    def match_prefix(self, req_id, token_ids) -> int:
        """For a request that holds no page yet: takes the longest run of cached pages that hold the
        beginning of ``token_ids`` (in every group) and returns how many tokens they cover.  At least the
        last token is left to be run."""
        if not self.prefix_caching:
            return 0
        req = self._requests[req_id]
        if any(req.tables) or req.tokens:
            raise AssertionError(f"request {req_id!r} already holds pages")
        page_size = self.groups[0].page_size
        limit = (len(token_ids) - 1) // page_size
        previous, found_pages = 0, []
        for idx in range(limit):
            tokens = tuple(token_ids[idx * page_size:(idx + 1) * page_size])
            content_hash = self._chain(previous, tokens)
            found = [pool.find(content_hash, tokens) for pool in self.pools]
            if any(page is None for page in found):
                break
            found_pages.append((content_hash, found))
            previous = content_hash
        for content_hash, found in found_pages:
            for gi, page in enumerate(found):
                self.pools[gi].share(page)
                req.tables[gi].append(page)
            req.hashes.append(content_hash)
        covered = len(found_pages) * page_size
        req.tokens = [int(t) for t in token_ids[:covered]]
        return covered

    def _publish(self, req: _Request, cached_after: int) -> None:
        page_size = self.groups[0].page_size
        if req.unknown_at is not None:   # a page is named only once all its tokens are known
            cached_after = min(cached_after, req.unknown_at)
        while len(req.hashes) < cached_after // page_size:
            idx = len(req.hashes)
            tokens = tuple(req.tokens[idx * page_size:(idx + 1) * page_size])
            content_hash = self._chain(req.hashes[-1] if req.hashes else 0, tokens)
            req.hashes.append(content_hash)
            for gi, pool in enumerate(self.pools):
                pool.publish(req.tables[gi][idx], content_hash, tokens)

    def commit(self, req_id, cached_after: int, tokens=None, last_unknown: bool = False) -> None:
        """After a step: ``cached_after`` tokens are in the cache (``tokens``: the ones this step ran,
        which the prefix cache needs to name the pages they filled; ``last_unknown``: the last of them
        was taken from the device and its value comes later, through ``amend``).  Pages of window groups
        that no later query can see are given back."""
        req = self._requests[req_id]
        req.fresh = False
        if self.prefix_caching:
            if tokens is None:
                raise ValueError("the prefix cache needs the tokens of every step")
            if last_unknown:
                if req.unknown_at is not None:
                    raise AssertionError(f"request {req_id!r}: a second token whose value is not known yet")
                req.unknown_at = len(req.tokens) + len(tokens) - 1
            req.tokens.extend(int(t) for t in tokens)
            if len(req.tokens) != cached_after:
                raise AssertionError(f"request {req_id!r}: {len(req.tokens)} tokens noted, {cached_after} in the cache")
            self._publish(req, cached_after)
        for gi, g in enumerate(self.groups):
            if g.window is None:
                continue
            first = self._first_page_needed(gi, cached_after)
            table = req.tables[gi]
            for idx in range(min(first, len(table))):
                if table[idx] >= 0:
                    self.pools[gi].give(table[idx])
                    table[idx] = -1

    def awaited_position(self, req_id) -> int | None:
        """The position whose token ``commit`` took as not yet known, if there is one."""
        return self._requests[req_id].unknown_at

    def amend(self, req_id, position: int, token: int) -> None:
        """The value of the token at ``position``, which ``commit`` took as not yet known."""
        if not self.prefix_caching:
            return
        req = self._requests[req_id]
        if req.unknown_at != position:
            raise AssertionError(f"request {req_id!r}: position {position} is not the one whose token is awaited "
                                 f"({req.unknown_at})")
        req.tokens[position] = int(token)
        req.unknown_at = None
        self._publish(req, len(req.tokens))

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
        """No page lost; every page held exactly as often as it is counted (more than once only through
        the prefix cache); none both free and held; same for slots."""
        for gi, (g, pool) in enumerate(zip(self.groups, self.pools)):
            held: dict[int, int] = {}
            for req in self._requests.values():
                for p in req.tables[gi]:
                    if p >= 0:
                        held[p] = held.get(p, 0) + 1
            if not self.prefix_caching:
                assert all(n == 1 for n in held.values()), f"group {gi}: a page is held twice"
            for p, n in held.items():
                assert pool.refs(p) == n, f"group {gi}: page {p} is held {n} times but counted {pool.refs(p)}"
            free = list(pool._free) + list(pool._cached)
            assert len(free) == len(set(free)), f"group {gi}: a page is free twice"
            assert not (set(free) & set(held)), f"group {gi}: a page is free and held"
            assert len(free) + len(held) == g.num_pages, f"group {gi}: {g.num_pages - len(free) - len(held)} page(s) lost"
            assert all(pool.refs(p) == 0 for p in free)
            for h, p in pool._by_hash.items():
                assert pool.hash_of(p) == h
        slots = [r.slot for r in self._requests.values()]
        assert len(slots) == len(set(slots)), "a state slot is held twice"
        assert len(slots) + self.slots.num_free == self.slots.num_slots, "a state slot is lost"
