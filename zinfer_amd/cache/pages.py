"""Page and slot bookkeeping of the cache: which pages are free, which request holds which.
Pure host code; it never touches a device."""
from __future__ import annotations

from typing import Dict, List

from ..errors import CacheFull, ZinferError


class PageAllocator:
    """Pages 0..num_pages-1 with a last-in-first-out free list, so that a page given back is
    the next one handed out (reuse happens early, which is what tests with few pages need).
    Handing out is all-or-nothing; a page is never held twice nor freed twice."""

    def __init__(self, num_pages: int):
        if num_pages < 0:
            raise ValueError("num_pages must not be negative")
        self.num_pages = num_pages
        self._free: List[int] = list(range(num_pages - 1, -1, -1))
        self._held = [False] * num_pages
        self.high_water = 0
        self.handed_out = 0          # pages handed out over the allocator's life

    @property
    def num_free(self) -> int:
        return len(self._free)

    @property
    def num_held(self) -> int:
        return self.num_pages - len(self._free)

    def alloc(self, n: int) -> List[int]:
        if n > len(self._free):
            raise CacheFull(f"CacheFull: {n} pages wanted, {len(self._free)} of "
                            f"{self.num_pages} free")
        out = []
        for _ in range(n):
            p = self._free.pop()
            assert not self._held[p], f"page {p} handed out twice"
            self._held[p] = True
            out.append(p)
        self.handed_out += n
        self.high_water = max(self.high_water, self.num_held)
        return out

    def free(self, pages) -> None:
        for p in pages:
            if not (0 <= p < self.num_pages) or not self._held[p]:
                raise ZinferError(f"page {p} freed but not held")
            self._held[p] = False
            self._free.append(p)

    def check(self) -> None:
        """Every page is either free or held, once."""
        assert len(set(self._free)) == len(self._free), "a page is on the free list twice"
        for p in self._free:
            assert not self._held[p], f"page {p} is free and held"
        assert sum(self._held) + len(self._free) == self.num_pages, "a page was lost"
