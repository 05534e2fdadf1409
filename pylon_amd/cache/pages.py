"""A pool of page ids with a last-in-first-out free list and a reference count per page.

The reference keeps the free list as a Python list used as a stack and lets a page
return to it when its handle object is collected
(/root/reference/src/pylon/kv/pool.py:45,65-75,10-16); here holding and giving back
are explicit, so a page given back twice, or one the pool never handed out, is an error
rather than a silent corruption.
"""
from __future__ import annotations

from typing import List


class OutOfPages(RuntimeError):
    """More pages were asked for than are free; nothing was taken."""


class PagePool:
    def __init__(self, num_pages: int) -> None:
        if num_pages < 1:
            raise ValueError("KV page pool must contain at least one page.")
        self.num_pages = num_pages
        # Pages come out 0, 1, 2, ... from a fresh pool; a page given back is the next out.
        self._free: List[int] = list(range(num_pages - 1, -1, -1))
        self._refs: List[int] = [0] * num_pages

    @property
    def free_pages(self) -> int:
        return len(self._free)

    @property
    def used_pages(self) -> int:
        return self.num_pages - len(self._free)

    def acquire(self, count: int) -> List[int]:
        if count < 0:
            raise ValueError("Requested page count must not be negative.")
        if count > len(self._free):
            raise OutOfPages(
                f"KV page pool needs {count} pages but only {len(self._free)} are free."
            )
        pages = [self._free.pop() for _ in range(count)]
        for page in pages:
            self._refs[page] = 1
        return pages

    def retain(self, page: int) -> None:
        """One more holder of a page that is already held."""
        self._check_id(page)
        if self._refs[page] < 1:
            raise RuntimeError(f"page {page} is free and cannot be retained")
        self._refs[page] += 1

    def release(self, page: int) -> None:
        """One holder less; the page goes back to the free list with the last one."""
        self._check_id(page)
        if self._refs[page] < 1:
            raise RuntimeError(f"page {page} was released more often than it was held")
        self._refs[page] -= 1
        if self._refs[page] == 0:
            self._free.append(page)

    def refcount(self, page: int) -> int:
        self._check_id(page)
        return self._refs[page]

    def check(self) -> None:
        """Raise unless every page is either free exactly once or held."""
        seen = set()
        for page in self._free:
            if page in seen:
                raise AssertionError(f"page {page} is on the free list twice")
            seen.add(page)
            if self._refs[page] != 0:
                raise AssertionError(f"page {page} is free but has {self._refs[page]} holders")
        for page in range(self.num_pages):
            if page not in seen and self._refs[page] < 1:
                raise AssertionError(f"page {page} is neither free nor held")

    def _check_id(self, page: int) -> None:
        if not isinstance(page, int) or not 0 <= page < self.num_pages:
            raise ValueError(f"page id {page!r} is not one of this pool's {self.num_pages} pages")
