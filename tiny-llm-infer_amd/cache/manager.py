"""The cache manager: keys and values in pages, a block table per request and
group, and slots for per-request state of fixed size.

A mixer states what it needs of the cache as a ``CacheNeed``.  Cache layers
with equal needs form a group; a group owns a pool of page ids, one device
tensor for keys and one for values, and one block table per request, so layers
that keep all keys and layers that keep a window of them do not share pages.
A window group gives a page back as soon as every slot of it lies before the
window of all tokens still to come; every group gives all of a request's pages
back when the request ends.  (The reference has one group and no window:
model/src/qwen3_kv_cache.cpp:14-44, engine/src/block_manager.cpp.)

Page layout on the device: keys ``[cache layer in group, page, kv head, slot,
head_dim]``, values ``[cache layer in group, page, kv head, head_dim, slot]``, so
that one head's part of a page is contiguous and each matrix-core operand is
contiguous along the index it is contracted over.  The block table of a
request maps ``position // page_size`` to a page id, -1 where no page is held.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, Hashable, List, Optional, Sequence, Tuple

from .pages import PageError, PagePool


class CacheFull(RuntimeError):
    """No pages (or state slots) are left for what was asked."""


@dataclass(frozen=True)
class CacheNeed:
    """What one mixer needs of the paged cache.  ``window`` None: all keys."""
    num_kv_heads: int
    head_dim: int
    window: Optional[int] = None


@dataclass(frozen=True)
class StateNeed:
    """Fixed-size state per request: ``shape`` elements of ``dtype`` (a torch dtype)."""
    shape: Tuple[int, ...]
    dtype: object


@dataclass
class GroupLayout:
    need: CacheNeed
    cache_layers: List[int]            # global cache layer ids, in group order
    pool: PagePool
    index: int = 0

    def local_layer(self, cache_layer: int) -> int:
        return self.cache_layers.index(cache_layer)


@dataclass
class RequestCache:
    """What one live request holds."""
    key: Hashable
    slot: int
    num_tokens: int = 0                               # tokens whose keys are in the cache
    tables: List[List[int]] = field(default_factory=list)   # per group: block -> page or -1
    reserved_tokens: int = 0                          # positions [0, reserved) are covered


def _blocks(tokens: int, page: int) -> int:
    return (tokens + page - 1) // page


class CacheManager:
    def __init__(self, needs: Sequence[Optional[CacheNeed]], page_size: int, num_pages: int,
                 max_requests: int):
        """``needs[i]`` is the need of cache layer i (None: that layer keeps nothing).
        Every group gets ``num_pages`` pages of ``page_size`` slots."""
        if page_size <= 0 or num_pages <= 0 or max_requests <= 0:
            raise ValueError("page_size, num_pages and max_requests must be positive")
        self.page_size = page_size
        self.num_pages = num_pages
        self.max_requests = max_requests
        self.groups: List[GroupLayout] = []
        self.group_of_layer: Dict[int, int] = {}
        by_need: Dict[CacheNeed, GroupLayout] = {}
        for layer, need in enumerate(needs):
            if need is None:
                continue
            g = by_need.get(need)
            if g is None:
                g = GroupLayout(need, [], PagePool(num_pages), index=len(self.groups))
                by_need[need] = g
                self.groups.append(g)
            g.cache_layers.append(layer)
            self.group_of_layer[layer] = g.index
        self._free_slots = list(range(max_requests - 1, -1, -1))   # pop() gives the lowest
        self._live: Dict[Hashable, RequestCache] = {}
        self.pages_taken_total = 0
        self.pages_returned_total = 0

    # ---- requests -------------------------------------------------------
    def live(self) -> List[Hashable]:
        return list(self._live)

    def get(self, key: Hashable) -> RequestCache:
        return self._live[key]

    def __contains__(self, key: Hashable) -> bool:
        return key in self._live

    def free_slots(self) -> int:
        return len(self._free_slots)

    def admit(self, key: Hashable) -> RequestCache:
        """Give a new request a state slot and empty block tables."""
        if key in self._live:
            raise ValueError(f"request {key!r} is already live")
        if not self._free_slots:
            raise CacheFull("no state slot is free")
        slot = self._free_slots.pop()
        rc = RequestCache(key=key, slot=slot, tables=[[] for _ in self.groups])
        self._live[key] = rc
        return rc

    # ---- pages ----------------------------------------------------------
    def _first_needed_block(self, g: GroupLayout, first_query_pos: int) -> int:
        """Lowest block a query at ``first_query_pos`` (and any later one) can read."""
        if g.need.window is None:
            return 0
        return max(0, first_query_pos - g.need.window + 1) // self.page_size

    def pages_needed(self, key: Hashable, new_total: int) -> List[int]:
        """Per group, pages that must be taken so that the request can run the
        tokens at positions [num_tokens, new_total)."""
        rc = self._live[key]
        out = []
        for gi, g in enumerate(self.groups):
            table = rc.tables[gi]
            first = self._first_needed_block(g, rc.num_tokens)
            need = 0
            for b in range(first, _blocks(new_total, self.page_size)):
                if b >= len(table) or table[b] < 0:
                    need += 1
            out.append(need)
        return out

    def can_reserve(self, key: Hashable, new_total: int) -> bool:
        return all(n <= g.pool.free_count
                   for n, g in zip(self.pages_needed(key, new_total), self.groups))

    def reserve(self, key: Hashable, new_total: int) -> None:
        """Take pages so that positions up to ``new_total`` can be written and
        everything a query in [num_tokens, new_total) reads is held.  All or
        nothing: CacheFull leaves the request as it was."""
        rc = self._live[key]
        if new_total < rc.num_tokens:
            raise ValueError("a request cannot shrink")
        if not self.can_reserve(key, new_total):
            raise CacheFull(f"not enough free pages to hold {new_total} tokens of {key!r}")
        for gi, g in enumerate(self.groups):
            table = rc.tables[gi]
            nb = _blocks(new_total, self.page_size)
            while len(table) < nb:
                table.append(-1)
            first = self._first_needed_block(g, rc.num_tokens)
            for b in range(first, nb):
                if table[b] < 0:
                    table[b] = g.pool.take()
                    self.pages_taken_total += 1
        rc.reserved_tokens = max(rc.reserved_tokens, new_total)

    def advance(self, key: Hashable, new_total: int) -> None:
        """Record that the tokens up to ``new_total`` are now in the cache and
        give back the pages of window groups that no later token can read."""
        rc = self._live[key]
        if new_total > rc.reserved_tokens:
            raise ValueError(f"{key!r}: {new_total} tokens were run but only "
                             f"{rc.reserved_tokens} were reserved")
        rc.num_tokens = new_total
        for gi, g in enumerate(self.groups):
            if g.need.window is None:
                continue
            table = rc.tables[gi]
            first = min(self._first_needed_block(g, new_total), len(table))
            for b in range(first):
                if table[b] >= 0:
                    g.pool.release(table[b])
                    self.pages_returned_total += 1
                    table[b] = -1

    def release(self, key: Hashable) -> None:
        """The request has ended (or is preempted): all it holds is given back,
        pages in reverse table order as the reference does
        (engine/src/block_manager.cpp:150-159)."""
        rc = self._live.pop(key)
        for gi, g in enumerate(self.groups):
            for page in reversed(rc.tables[gi]):
                if page >= 0:
                    g.pool.release(page)
                    self.pages_returned_total += 1
            rc.tables[gi] = []
        self._free_slots.append(rc.slot)
        self._free_slots.sort(reverse=True)

    # ---- inspection -----------------------------------------------------
    def free_pages(self) -> List[int]:
        return [g.pool.free_count for g in self.groups]

    def check(self) -> None:
        """No page lost, held twice or freed twice; slots likewise."""
        for gi, g in enumerate(self.groups):
            g.pool.check()
            held: Dict[int, int] = {}
            for rc in self._live.values():
                for page in rc.tables[gi]:
                    if page >= 0:
                        held[page] = held.get(page, 0) + 1
            for page in range(g.pool.num_pages):
                if g.pool.ref_count(page) != held.get(page, 0):
                    raise PageError(f"group {gi} page {page}: pool counts "
                                    f"{g.pool.ref_count(page)} holders, tables show {held.get(page, 0)}")
        slots = [rc.slot for rc in self._live.values()] + self._free_slots
        if sorted(slots) != list(range(self.max_requests)):
            raise PageError("state slots are lost or held twice")
