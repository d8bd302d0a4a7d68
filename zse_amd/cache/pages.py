"""A pool of page ids with a free list.

The reference's ``BlockPool`` is one slab whose block holds every layer, with a
FIFO free list and reference counts (cache/block_pool.py:61-122, 189-227).
Here a pool belongs to one group of layers, hands out plain ids (the slabs are
the mixers' business), keeps no counts since nothing is shared, and reuses the
page freed last first, so reuse is immediate.
"""
from __future__ import annotations

from typing import List, Optional


class OutOfPages(RuntimeError):
    pass


class PagePool:
    def __init__(self, num_pages: int, first_id: int = 0):
        """``num_pages`` pages with the ids ``first_id`` .. ``first_id + num_pages - 1``.  An owner
        of the pages' memory that keeps a page of its own in front of them (one that is never
        handed out, for table entries that name no page) starts the ids at 1."""
        if num_pages <= 0:
            raise ValueError(f"a pool needs at least one page, got {num_pages}")
        if first_id < 0:
            raise ValueError("page ids are not negative")
        self.num_pages = int(num_pages)
        self.first_id = int(first_id)
        last = self.first_id + self.num_pages - 1
        self._free: List[int] = list(range(last, self.first_id - 1, -1))   # pop() gives the first id first
        self._owner: List[Optional[object]] = [None] * (last + 1)

    @property
    def free_pages(self) -> int:
        return len(self._free)

    @property
    def used_pages(self) -> int:
        return self.num_pages - len(self._free)

    def alloc(self, owner) -> int:
        if owner is None:
            raise ValueError("a page needs an owner")
        if not self._free:
            raise OutOfPages(f"no free page among {self.num_pages}")
        p = self._free.pop()
        assert self._owner[p] is None, f"page {p} was free and owned"
        self._owner[p] = owner
        return p

    def free(self, page: int, owner) -> None:
        if not (self.first_id <= page < self.first_id + self.num_pages):
            raise ValueError(f"page {page} is not in the pool")
        if self._owner[page] is None:
            raise RuntimeError(f"page {page} freed twice")
        if self._owner[page] != owner:
            raise RuntimeError(f"page {page} belongs to {self._owner[page]!r}, not {owner!r}")
        self._owner[page] = None
        self._free.append(page)

    def owner(self, page: int):
        return self._owner[page]

    def check(self) -> None:
        """Every page is either free or owned, never both, never twice on the free list."""
        free = set(self._free)
        if len(free) != len(self._free):
            raise AssertionError("a page is on the free list twice")
        for p in range(self.first_id, self.first_id + self.num_pages):
            if (p in free) == (self._owner[p] is not None):
                raise AssertionError(f"page {p}: free={p in free}, owner={self._owner[p]!r}")
