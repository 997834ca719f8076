"""Free list of cache pages.

As in the reference's BlockManager (src/engine/block_manager.cpp:5-36) the list
is LIFO over ids 0..N-1: the first page handed out is N-1 and a page given back
is the next one handed out, so freed pages are used again at once.  Unlike
there, a page cannot be freed twice or freed without having been handed out.
"""
from __future__ import annotations

from typing import List


class OutOfPages(RuntimeError):
    pass


class PagePool:
    def __init__(self, num_pages: int):
        if num_pages < 0:
            raise ValueError("num_pages must not be negative")
        self.num_pages = num_pages
        self._free: List[int] = list(range(num_pages))
        self._held = [False] * num_pages

    @property
    def num_free(self) -> int:
        return len(self._free)

    def allocate(self) -> int:
        if not self._free:
            raise OutOfPages("no free cache page (pool of %d)" % self.num_pages)
        page = self._free.pop()
        self._held[page] = True
        return page

    def free(self, page: int) -> None:
        if not (0 <= page < self.num_pages):
            raise ValueError("page %r is not in the pool of %d" % (page, self.num_pages))
        if not self._held[page]:
            raise ValueError("page %d is freed but not held" % page)
        self._held[page] = False
        self._free.append(page)

    def held(self) -> List[int]:
        return [p for p, h in enumerate(self._held) if h]
