"""Free list and reference counts of one group's pages.

Reference: ``BlockAllocator`` (somi_inference/core/paged_attention.py:24-59): a
free stack popped from the end (so freed pages are used again first) and a
reference count per page.  The reference lets an empty pool raise a bare
``IndexError`` (:37); here that is :class:`OutOfPages`, and freeing a page that
is not held is an error instead of a negative count.
"""

from __future__ import annotations


class OutOfPages(RuntimeError):
    """The pool has no free page left."""


class CacheError(RuntimeError):
    """A page or request was used against the manager's rules (double free, unknown id...)."""


class PagePool:
    def __init__(self, num_pages: int) -> None:
        if num_pages < 1:
            raise ValueError(f"a page pool needs at least one page, got {num_pages}")
        self.num_pages = int(num_pages)
        self._free = list(range(self.num_pages))
        self._refs = [0] * self.num_pages

    @property
    def num_free(self) -> int:
        return len(self._free)

    def allocate(self) -> int:
        if not self._free:
            raise OutOfPages(f"all {self.num_pages} pages are in use")
        page = self._free.pop()
        if self._refs[page] != 0:
            raise CacheError(f"page {page} was on the free list while still referenced")
        self._refs[page] = 1
        return page

    def retain(self, page: int) -> None:
        if self._refs[page] < 1:
            raise CacheError(f"page {page} is not held")
        self._refs[page] += 1

    def release(self, page: int) -> None:
        if not 0 <= page < self.num_pages or self._refs[page] < 1:
            raise CacheError(f"page {page} is released but not held")
        self._refs[page] -= 1
        if self._refs[page] == 0:
            self._free.append(page)

    def refcount(self, page: int) -> int:
        return self._refs[page]

    def free_pages(self) -> list[int]:
        return list(self._free)
