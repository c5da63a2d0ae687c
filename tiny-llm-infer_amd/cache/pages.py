"""Page ids of one pool: which are free, which are held and how often.

As in the reference's block manager the lowest free id is handed out first
(an ordered set there, engine/src/block_manager.cpp:66-85; a heap here), which
makes allocation deterministic, and a page returns to the free set when its
reference count reaches zero (engine/src/block_manager.cpp:142-148).  Unlike
the reference, releasing a page that is not held is an error, not a no-op.
"""
from __future__ import annotations

import heapq
from typing import List


class PageError(RuntimeError):
    pass


class PagePool:
    def __init__(self, num_pages: int):
        if num_pages < 0:
            raise ValueError("num_pages must not be negative")
        self.num_pages = num_pages
        self._free: List[int] = list(range(num_pages))
        heapq.heapify(self._free)
        self._refs = [0] * num_pages

    @property
    def free_count(self) -> int:
        return len(self._free)

    @property
    def held_count(self) -> int:
        return self.num_pages - len(self._free)

    def ref_count(self, page: int) -> int:
        return self._refs[page]

    def take(self) -> int:
        """Hand out the lowest free page id; PageError if none is left."""
        if not self._free:
            raise PageError("the page pool is exhausted")
        page = heapq.heappop(self._free)
        assert self._refs[page] == 0
        self._refs[page] = 1
        return page

    def share(self, page: int) -> None:
        if self._refs[page] <= 0:
            raise PageError(f"page {page} is not held and cannot be shared")
        self._refs[page] += 1

    def release(self, page: int) -> None:
        if page < 0 or page >= self.num_pages:
            raise PageError(f"page id {page} is outside the pool")
        if self._refs[page] <= 0:
            raise PageError(f"page {page} is released but not held")
        self._refs[page] -= 1
        if self._refs[page] == 0:
            heapq.heappush(self._free, page)

    def check(self) -> None:
        """Every page is either free exactly once or held: none lost, none twice."""
        free = sorted(self._free)
        if len(set(free)) != len(free):
            raise PageError("a page is in the free set twice")
        for p in range(self.num_pages):
            if (self._refs[p] == 0) != (p in set(free)):
                raise PageError(f"page {p}: reference count {self._refs[p]} disagrees with the free set")
