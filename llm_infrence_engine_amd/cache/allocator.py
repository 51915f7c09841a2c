"""Page ids of one pool: a free list with reference counts.  No tensors here.

Page 0 is the null page: never handed out, it pads block tables and stands for pages a window has
passed, so a table entry can always be dereferenced (src/miniserve/paged.py:34, 68).  Fresh pages come
out in ascending order and a page given back goes to the end of the list (paged.py:85-111), so a small
pool reuses pages soon.  The reference's prefix-hash map and eviction list (paged.py:114-122) are a
sharing policy and not part of this allocator; the reference counts that sharing would need are kept.
"""
from __future__ import annotations

from collections import deque

NULL_PAGE = 0


class OutOfPages(Exception):
    """No free page is left in a pool."""


class PageAllocator:
    def __init__(self, num_pages: int):
        """``num_pages`` usable pages with ids 1..num_pages (the null page comes on top)."""
        if num_pages < 1:
            raise ValueError("a pool needs at least one page beside the null page")
        self.num_pages = num_pages
        self.ref = [0] * (num_pages + 1)
        self.grants = [0] * (num_pages + 1)     # how often each page has been handed out so far
        self._free = deque(range(1, num_pages + 1))

    @property
    def capacity(self) -> int:
        return self.num_pages

    def num_free(self) -> int:
        return len(self._free)

    def num_in_use(self) -> int:
        return self.num_pages - len(self._free)

    def allocate(self) -> int:
        if not self._free:
            raise OutOfPages()
        p = self._free.popleft()
        self.ref[p] = 1
        self.grants[p] += 1
        return p

    def pages_granted_again(self) -> int:
        """Pages that have been handed out more than once: a small pool in use shows reuse here."""
        return sum(1 for n in self.grants if n > 1)

    def incref(self, p: int) -> None:
        if p == NULL_PAGE or self.ref[p] <= 0:
            raise ValueError(f"page {p} is not held by anyone and cannot be shared")
        self.ref[p] += 1

    def decref(self, p: int) -> None:
        if p == NULL_PAGE or not 0 < p <= self.num_pages:
            raise ValueError(f"page {p} is not a page of this pool")
        if self.ref[p] <= 0:
            raise ValueError(f"page {p} given back more often than it was taken")
        self.ref[p] -= 1
        if self.ref[p] == 0:
            self._free.append(p)

    def check_invariants(self) -> None:
        """Every page is either free (count 0, once in the list) or held (count > 0, not in the list)."""
        free = list(self._free)
        assert len(free) == len(set(free)), "a page is in the free list twice"
        fs = set(free)
        assert NULL_PAGE not in fs and self.ref[NULL_PAGE] == 0, "the null page was handed out or freed"
        for p in range(1, self.num_pages + 1):
            assert self.ref[p] >= 0
            assert (self.ref[p] == 0) == (p in fs), f"page {p}: count {self.ref[p]} but {'in' if p in fs else 'not in'} the free list"
