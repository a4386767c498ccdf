"""The page allocator: a free list of page numbers and a map of which are in use.

reference: KvBlockAllocator (app/server.cpp:96-128): a FIFO free list of slot numbers and an
`in_use_` array; `Acquire()` pops the front, `Release(slot)` refuses a number out of range or not
in use.  There a slot is one request's whole cache; here a page holds `page_size` positions, a
request holds as many as it needs, and `alloc(n)` gives all n or none.  The list is FIFO, so a
page that was just given back is the last to be handed out again; with few pages it still comes
round quickly, which is what the tests of reuse lean on.
"""
from __future__ import annotations

from collections import deque

from ..errors import invalid_argument


class PageAllocator:
    def __init__(self, num_pages: int):
        if num_pages <= 0:
            raise invalid_argument("a page pool needs at least one page")
        self.num_pages = num_pages
        self._free = deque(range(num_pages))
        self._in_use = bytearray(num_pages)

    @property
    def num_free(self) -> int:
        return len(self._free)

    @property
    def num_used(self) -> int:
        return self.num_pages - len(self._free)

    def alloc(self, count: int) -> list[int] | None:
        """`count` pages, or None when fewer are free (then nothing is taken)."""
        if count < 0:
            raise invalid_argument("cannot allocate a negative number of pages")
        if count > len(self._free):
            return None
        pages = [self._free.popleft() for _ in range(count)]
        for page in pages:
            self._in_use[page] = 1
        return pages

    def release(self, pages) -> None:
        """Gives pages back.  A page out of range or not in use is refused, and then none of
        the call's pages is given back."""
        pages = list(pages)
        seen = set()
        for page in pages:
            if not 0 <= page < self.num_pages:
                raise invalid_argument(f"page {page} is outside the pool of {self.num_pages}")
            if not self._in_use[page] or page in seen:
                raise invalid_argument(f"page {page} is freed twice")
            seen.add(page)
        for page in pages:
            self._in_use[page] = 0
            self._free.append(page)

    def in_use(self, page: int) -> bool:
        return bool(self._in_use[page])

    def free_pages(self) -> list[int]:
        return list(self._free)
