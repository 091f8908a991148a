"""A pool of cache pages with a free list."""
from __future__ import annotations


class OutOfPages(RuntimeError):
    """The pool cannot give as many pages as were asked for."""


class BlockPool:
    """Page ids 0..num_pages-1.  ``allocate`` is all-or-nothing; freed pages go
    on top of a stack and are handed out again first, so a page is reused as
    soon as possible.

    Reference: PageManager with ``_free_list`` (push_back / pop_back),
    ``allocate()`` returning INVALID_PAGE_ID when empty, ``free(id)``,
    ``used_count()`` (src/core/runtime/KVCache.h:81-100, :164-167).  There a
    page belongs to one layer of one sequence and is never given back
    (``clear`` exists at :245-253, :445-455 but nothing calls it).
    """

    def __init__(self, num_pages: int):
        if num_pages <= 0:
            raise ValueError(f"a pool needs at least one page, got {num_pages}")
        self.num_pages = int(num_pages)
        self._free = list(range(self.num_pages - 1, -1, -1))  # pop() gives 0 first
        self._used = [False] * self.num_pages

    @property
    def num_free(self) -> int:
        return len(self._free)

    @property
    def num_used(self) -> int:
        return self.num_pages - len(self._free)

    def allocate(self, n: int) -> list[int]:
        if n < 0:
            raise ValueError("negative page count")
        if n > len(self._free):
            raise OutOfPages(f"{n} pages wanted, {len(self._free)} of {self.num_pages} free")
        out = [self._free.pop() for _ in range(n)]
        for p in out:
            self._used[p] = True
        return out

    def free(self, pages) -> None:
        for p in pages:
            if not 0 <= p < self.num_pages:
                raise ValueError(f"page {p} is not of this pool")
            if not self._used[p]:
                raise ValueError(f"page {p} freed twice")
            self._used[p] = False
            self._free.append(p)

    def check(self) -> None:
        """Raises AssertionError if a page is lost or held twice."""
        assert len(set(self._free)) == len(self._free), "a page is on the free list twice"
        assert all(not self._used[p] for p in self._free), "a free page is marked used"
        assert sum(self._used) + len(self._free) == self.num_pages, "a page is lost"
