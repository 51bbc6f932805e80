"""The page pool: which pages are free, which are held.

Role of `BlockManager`'s free list in the reference (python/infinilm/llm/cache_manager.py:74-120):
pages leave the free list from its front and return to its back, so the order of reuse is
first-freed first-reused and a replay is deterministic.  A page is held by exactly one owner here
(no prefix sharing); holding twice or freeing twice is an error, not a silent no-op.
"""
from __future__ import annotations

from collections import deque
from typing import List


class CacheError(RuntimeError):
    pass


class OutOfPages(CacheError):
    """The pool cannot give the pages asked for; nothing was taken."""


class PagePool:
    def __init__(self, num_pages: int):
        if num_pages <= 0:
            raise CacheError(f"a page pool needs at least one page, got {num_pages}")
        self.num_pages = int(num_pages)
        self._free = deque(range(self.num_pages))
        self._held = [False] * self.num_pages
        self.high_water = 0

    @property
    def num_free(self) -> int:
        return len(self._free)

    @property
    def num_held(self) -> int:
        return self.num_pages - len(self._free)

    def take(self, n: int) -> List[int]:
        """n pages, or OutOfPages with nothing taken."""
        if n < 0:
            raise CacheError(f"cannot take {n} pages")
        if n > len(self._free):
            raise OutOfPages(f"{n} pages asked, {len(self._free)} free of {self.num_pages}")
        out = [self._free.popleft() for _ in range(n)]
        for p in out:
            if self._held[p]:
                raise CacheError(f"page {p} was on the free list while held")
            self._held[p] = True
        self.high_water = max(self.high_water, self.num_held)
        return out

    def give_back(self, pages) -> None:
        for p in pages:
            if not 0 <= p < self.num_pages:
                raise CacheError(f"page {p} is not of this pool")
            if not self._held[p]:
                raise CacheError(f"page {p} given back twice")
            self._held[p] = False
            self._free.append(p)

    def check(self) -> None:
        """Every page is either free once or held: none lost, none twice."""
        free = list(self._free)
        if len(set(free)) != len(free):
            raise CacheError("a page is on the free list twice")
        free_set = set(free)
        for p in range(self.num_pages):
            if self._held[p] == (p in free_set):
                raise CacheError(f"page {p} is {'held and free' if self._held[p] else 'neither held nor free'}")
