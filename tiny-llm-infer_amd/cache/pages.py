"""Page ids of one pool: which are free, which are held and how often.

As in the reference's block manager the lowest free id is handed out first
(an ordered set there, engine/src/block_manager.cpp:66-85; a heap here), which
makes allocation deterministic, and a page returns to the free set when its
reference count reaches zero (engine/src/block_manager.cpp:142-148).  A free
page keeps its contents, so a page that the prefix cache still knows can be
taken back by id (``revive``) until it is handed out for something else.
Unlike the reference, releasing a page that is not held is an error, not a
no-op.
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
        self._heap: List[int] = list(range(num_pages))     # may hold ids that are held (lazy deletion),
        heapq.heapify(self._heap)                           # but every id at most once
        self._in_heap = [True] * num_pages
        self._is_free = [True] * num_pages
        self._free_count = num_pages
        self._refs = [0] * num_pages

    @property
    def free_count(self) -> int:
        return self._free_count

    @property
    def held_count(self) -> int:
        return self.num_pages - self._free_count

    def ref_count(self, page: int) -> int:
        return self._refs[page]

    def is_free(self, page: int) -> bool:
        return self._is_free[page]

    def take(self) -> int:
        """Hand out the lowest free page id; PageError if none is left."""
        if self._free_count == 0:
            raise PageError("the page pool is exhausted")
        while True:
            page = heapq.heappop(self._heap)
            self._in_heap[page] = False
            if self._is_free[page]:
                break
        assert self._refs[page] == 0
        self._is_free[page] = False
        self._free_count -= 1
        self._refs[page] = 1
        return page

    def revive(self, page: int) -> None:
        """Take a particular free page (its contents are wanted again)."""
        if not self._is_free[page]:
            raise PageError(f"page {page} is not free")
        self._is_free[page] = False          # its heap entry stays: skipped by take(), used again by release()
        self._free_count -= 1
        self._refs[page] = 1

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
            self._is_free[page] = True
            self._free_count += 1
            if not self._in_heap[page]:          # (a revived page's entry is still there)
                heapq.heappush(self._heap, page)
                self._in_heap[page] = True

    def check(self) -> None:
        """Every page is either free or held, the count is right, and every free
        page can still be found: none lost, none twice."""
        if sum(self._is_free) != self._free_count:
            raise PageError("the count of free pages is wrong")
        if len(self._heap) != sum(self._in_heap) or len(set(self._heap)) != len(self._heap):
            raise PageError("a page id is queued twice")
        reachable = set(self._heap)
        for p in range(self.num_pages):
            if self._is_free[p] != (self._refs[p] == 0):
                raise PageError(f"page {p}: reference count {self._refs[p]} disagrees with the free set")
            if self._is_free[p] and p not in reachable:
                raise PageError(f"free page {p} is lost")
