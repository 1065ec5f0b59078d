"""Free lists: pages of a cache pool and slots for per-request state.

Pure bookkeeping, no tensors (`pyre/paged_cache.py:40-92` is the reference's
allocator; this one has the same stack discipline and the same errors, without
reference counts, because nothing here shares pages between requests).
"""

from __future__ import annotations


class OutOfPages(MemoryError):
    """The pool has no free page (`pyre/paged_cache.py:62-67`)."""


class PageAllocator:
    """A stack of free ids over ``range(num_pages)``: the page freed last is the
    page handed out next, so a pool under pressure re-uses pages at once."""

    def __init__(self, num_pages: int, what: str = "page"):
        if num_pages < 0:
            raise ValueError("num_pages must not be negative")
        self.num_pages = num_pages
        self.what = what
        self._free = list(range(num_pages - 1, -1, -1))  # pop() yields 0 first
        self._used = [False] * num_pages

    @property
    def num_free(self) -> int:
        return len(self._free)

    @property
    def num_used(self) -> int:
        return self.num_pages - len(self._free)

    def allocate(self) -> int:
        if not self._free:
            raise OutOfPages(f"{self.what} pool exhausted ({self.num_pages} {self.what}s all in use)")
        p = self._free.pop()
        self._used[p] = True
        return p

    def allocate_many(self, n: int) -> list[int]:
        """All n or none."""
        if n > len(self._free):
            raise OutOfPages(
                f"{self.what} pool exhausted ({n} needed, {len(self._free)} of {self.num_pages} free)")
        return [self.allocate() for _ in range(n)]

    def free(self, p: int) -> None:
        if not (0 <= p < self.num_pages) or not self._used[p]:
            raise ValueError(f"double free or freeing unallocated {self.what} {p}")
        self._used[p] = False
        self._free.append(p)

    def is_used(self, p: int) -> bool:
        return self._used[p]
