"""The page pool: which pages are free, which are held, and which keep a finished prefix.

Role of `BlockManager` in the reference (python/infinilm/llm/cache_manager.py:74-156): pages leave
the free list from its front and return to its back, so the order of reuse is first-freed
first-reused and a replay is deterministic; a page whose tokens are all computed can be published
under a key of its content (the reference chains xxh3 hashes, python/infinilm/llm/prefix_cache.py:15-28)
and then be shared by requests that begin with the same tokens.

A page here is in exactly one of three places:
  free   on the free list, content meaningless;
  held   in the block tables of `refs` requests (more than one only for published pages, which
         nobody writes any more);
  idle   published, held by nobody: its content stays until the pool needs the page; idle pages are
         taken after the free ones, least recently released first.
Holding what is not held, freeing twice or publishing twice is an error, not a silent no-op.
"""
from __future__ import annotations

from collections import OrderedDict, deque
from typing import Dict, List, Optional


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
        self._refs = [0] * self.num_pages
        self._key: List[Optional[bytes]] = [None] * self.num_pages
        self._index: Dict[bytes, int] = {}            # content key -> page
        self._idle: "OrderedDict[int, None]" = OrderedDict()
        self.high_water = 0
        self.evictions = 0

    @property
    def num_free(self) -> int:
        """Pages a request can still get: the free ones and the idle ones."""
        return len(self._free) + len(self._idle)

    @property
    def num_idle(self) -> int:
        return len(self._idle)

    @property
    def num_held(self) -> int:
        return self.num_pages - len(self._free) - len(self._idle)

    def take(self, n: int) -> List[int]:
        """n pages for one owner, or OutOfPages with nothing taken."""
        if n < 0:
            raise CacheError(f"cannot take {n} pages")
        if n > self.num_free:
            raise OutOfPages(f"{n} pages asked, {self.num_free} free of {self.num_pages}")
        out = []
        for _ in range(n):
            if self._free:
                p = self._free.popleft()
            else:
                p, _ = self._idle.popitem(last=False)     # the longest idle one loses its content
                del self._index[self._key[p]]
                self._key[p] = None
                self.evictions += 1
            if self._refs[p] != 0:
                raise CacheError(f"page {p} was free while held")
            self._refs[p] = 1
            out.append(p)
        self.high_water = max(self.high_water, self.num_held)
        return out

    def give_back(self, pages) -> None:
        """One owner less for each page; a page nobody holds goes to the idle ones if it is published,
        else to the back of the free list."""
        for p in pages:
            if not 0 <= p < self.num_pages:
                raise CacheError(f"page {p} is not of this pool")
            if self._refs[p] <= 0:
                raise CacheError(f"page {p} given back twice")
            self._refs[p] -= 1
            if self._refs[p] == 0:
                if self._key[p] is not None:
                    self._idle[p] = None
                else:
                    self._free.append(p)

    # ---- published pages --------------------------------------------------------------------------
    def publish(self, page: int, key: bytes) -> bool:
        """Makes a held page findable under the key of its content.  False (and nothing changes) if
        another page already has this content."""
        if self._refs[page] <= 0:
            raise CacheError(f"page {page} is published while nobody holds it")
        if self._key[page] is not None:
            raise CacheError(f"page {page} is published twice")
        if key in self._index:
            return False
        self._key[page] = key
        self._index[key] = page
        return True

    def lookup(self, key: bytes) -> Optional[int]:
        return self._index.get(key)

    def share(self, page: int) -> None:
        """One more owner for a published page (held or idle)."""
        if self._key[page] is None:
            raise CacheError(f"page {page} is not published: it cannot be shared")
        if self._refs[page] == 0:
            del self._idle[page]
        self._refs[page] += 1
        self.high_water = max(self.high_water, self.num_held)

    def is_published(self, page: int) -> bool:
        return self._key[page] is not None

    def refs(self, page: int) -> int:
        return self._refs[page]

    def check(self) -> None:
        """Every page is free once, idle once or held; the index holds exactly the published pages."""
        free = list(self._free)
        if len(set(free)) != len(free):
            raise CacheError("a page is on the free list twice")
        free_set = set(free)
        for p in range(self.num_pages):
            places = (p in free_set) + (p in self._idle) + (self._refs[p] > 0)
            if places != 1:
                raise CacheError(f"page {p} is in {places} of the places free / idle / held")
            if (p in free_set) and self._key[p] is not None:
                raise CacheError(f"page {p} is free but still published")
            if (p in self._idle) and self._key[p] is None:
                raise CacheError(f"page {p} is idle without a key")
            if self._key[p] is not None and self._index.get(self._key[p]) != p:
                raise CacheError(f"page {p}'s key is not in the index")
        if len(self._index) != sum(k is not None for k in self._key):
            raise CacheError("the index holds keys of pages that are not published")
