"""A fixed pool of page ids with reference counts."""

from __future__ import annotations


class OutOfPages(RuntimeError):
    """The pool has no free page left for what was asked."""


class PageAllocator:
    """Hands out page ids 0..num_pages-1 and takes them back.

    Semantics follow the reference's BlockAllocator (include/engine/block_allocator.hpp:14-72):
    the first ``allocate()`` returns 0, then 1, ...; a freed id is the next one handed out
    (last in, first out), so reuse is immediate; reference counts let two holders share a page;
    freeing a free page and adding a reference to a free page are errors.
    """

    def __init__(self, num_pages: int):
        if num_pages < 0:
            raise ValueError("PageAllocator: num_pages must be non-negative")
        self._free = list(range(num_pages - 1, -1, -1))
        self._refs = [0] * num_pages
        self._issued = [0] * num_pages  # how often each page has been handed out

    @property
    def num_pages(self) -> int:
        return len(self._refs)

    @property
    def num_free(self) -> int:
        return len(self._free)

    def allocate(self) -> int:
        if not self._free:
            raise OutOfPages("PageAllocator: out of pages")
        page = self._free.pop()
        self._refs[page] = 1
        self._issued[page] += 1
        return page

    def incref(self, page: int) -> None:
        if self._refs[page] == 0:
            raise RuntimeError(f"PageAllocator: incref on free page {page}")
        self._refs[page] += 1

    def free(self, page: int) -> None:
        if not 0 <= page < len(self._refs):
            raise RuntimeError(f"PageAllocator: page {page} is not in the pool")
        if self._refs[page] == 0:
            raise RuntimeError(f"PageAllocator: double free of page {page}")
        self._refs[page] -= 1
        if self._refs[page] == 0:
            self._free.append(page)

    def ref_count(self, page: int) -> int:
        return self._refs[page]

    @property
    def pages_issued(self) -> int:
        """How many times ``allocate`` has handed out a page since the pool was made."""
        return sum(self._issued)

    def pages_issued_again(self) -> list:
        """Ids of the pages that have been handed out more than once."""
        return [p for p, n in enumerate(self._issued) if n > 1]
