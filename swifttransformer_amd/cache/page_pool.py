"""A pool of cache pages with a free list.

The reference library has no allocator; its example driver hands out block ids
from a counter and never takes one back (src/examples/lib/inference_batch.cc:58-66),
exiting when they run out (:61-64).  Here pages return to a LIFO free list, so a
page given back is the next one handed out, and running out is an exception the
scheduler answers."""
from __future__ import annotations

from typing import List


class OutOfPages(RuntimeError):
    pass


class PagePool:
    def __init__(self, num_pages: int):
        if num_pages < 1:
            raise ValueError("a pool needs at least one page")
        self.num_pages = num_pages
        self._free: List[int] = list(range(num_pages - 1, -1, -1))   # pop() yields 0,1,2,...
        self._held = [False] * num_pages

    @property
    def num_free(self) -> int:
        return len(self._free)

    def alloc(self, n: int) -> List[int]:
        """n pages, or OutOfPages with nothing taken."""
        if n < 0:
            raise ValueError("negative page count")
        if n > len(self._free):
            raise OutOfPages(f"{n} pages wanted, {len(self._free)} free of {self.num_pages}")
        out = [self._free.pop() for _ in range(n)]
        for p in out:
            self._held[p] = True
        return out

    def free(self, pages) -> None:
        for p in pages:
            if not 0 <= p < self.num_pages:
                raise ValueError(f"page {p} is not of this pool")
            if not self._held[p]:
                raise ValueError(f"page {p} is freed twice")
            self._held[p] = False
            self._free.append(p)

    def is_held(self, page: int) -> bool:
        return self._held[page]
