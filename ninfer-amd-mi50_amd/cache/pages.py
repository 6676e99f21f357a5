"""Page allocator of one cache group.

Pages are handed out from a LIFO free list, so a page that was just given
back is the next one used again. Counters say how many pages were ever
handed out, given back, and handed out a second time. The reference has no
pages: it keeps one contiguous slab per (layer, sequence slot) and gives
nothing back (src/runtime/kv_cache.cpp:14-22).
"""
from __future__ import annotations

from typing import List


class OutOfPages(RuntimeError):
    """A reservation needs more pages than the pool has free."""


class PageAllocator:
    def __init__(self, num_pages: int):
        if num_pages < 1:
            raise ValueError(f"a page pool needs at least one page, got {num_pages}")
        self.num_pages = num_pages
        self._free: List[int] = list(range(num_pages - 1, -1, -1))  # pop() gives 0 first
        self._held = [False] * num_pages
        self._used_before = [False] * num_pages
        self.allocated = 0
        self.freed = 0
        self.reused = 0
        self.peak_in_use = 0

    @property
    def free_pages(self) -> int:
        return len(self._free)

    @property
    def in_use(self) -> int:
        return self.num_pages - len(self._free)

    def alloc(self, n: int) -> List[int]:
        """n pages, or OutOfPages with nothing taken."""
        if n > len(self._free):
            raise OutOfPages(f"need {n} pages, {len(self._free)} of {self.num_pages} are free")
        out = []
        for _ in range(n):
            p = self._free.pop()
            assert not self._held[p], f"page {p} handed out twice"
            self._held[p] = True
            if self._used_before[p]:
                self.reused += 1
            self._used_before[p] = True
            out.append(p)
        self.allocated += n
        self.peak_in_use = max(self.peak_in_use, self.in_use)
        return out

    def free(self, pages: List[int]) -> None:
        for p in pages:
            if not (0 <= p < self.num_pages) or not self._held[p]:
                raise RuntimeError(f"page {p} given back but not held")
            self._held[p] = False
            self._free.append(p)
        self.freed += len(pages)

    def is_held(self, page: int) -> bool:
        return 0 <= page < self.num_pages and self._held[page]

    def check(self) -> None:
        """Every page is either free or held, never both, never twice."""
        assert len(set(self._free)) == len(self._free), "a page is on the free list twice"
        for p in self._free:
            assert not self._held[p], f"page {p} is free and held"
        assert sum(self._held) + len(self._free) == self.num_pages, "a page was lost"
