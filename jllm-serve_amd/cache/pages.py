"""A pool of page ids: free list and reference counts, nothing else.

The reference's pool hands out block ids from a free list, counts references and raises when every
block is referenced (kv/KvPool.java:249-302, kv/KvPoolExhausted.java:4-8). The prefix tree and the eviction of
cached pages live beside this class (cache/prefix.py, driven by the cache manager); the spill tiers of the
reference's pool are not part of this engine. The contract kept here is: a page is either free or
held, ``alloc`` never returns a held page, ``release`` of the last reference makes it free at once.
"""
from __future__ import annotations

from typing import List


class OutOfPages(RuntimeError):
    """No free page (kv/KvPoolExhausted.java). The scheduler decides what happens next."""


class PagePool:
    def __init__(self, num_pages: int, page_tokens: int):
        if num_pages < 1 or page_tokens < 1:
            raise ValueError(f"a pool needs at least one page of at least one token, got {num_pages} x {page_tokens}")
        self.num_pages = num_pages
        self.page_tokens = page_tokens
        self._free: List[int] = list(range(num_pages - 1, -1, -1))  # pop() gives 0 first
        self._refs = [0] * num_pages
        self.high_water = 0
        self.allocations = 0

    @property
    def free_pages(self) -> int:
        return len(self._free)

    @property
    def used_pages(self) -> int:
        return self.num_pages - len(self._free)

    def alloc(self) -> int:
        if not self._free:
            raise OutOfPages(f"the KV pool is full: all {self.num_pages} pages of {self.page_tokens} positions are "
                             "in use by running sequences")
        p = self._free.pop()
        assert self._refs[p] == 0, f"page {p} was on the free list while referenced"
        self._refs[p] = 1
        self.allocations += 1
        self.high_water = max(self.high_water, self.used_pages)
        return p

    def retain(self, page: int) -> None:
        if self._refs[page] <= 0:
            raise ValueError(f"page {page} is not held")
        self._refs[page] += 1

    def release(self, page: int) -> None:
        if not 0 <= page < self.num_pages or self._refs[page] <= 0:
            raise ValueError(f"page {page} released but not held")
        self._refs[page] -= 1
        if self._refs[page] == 0:
            self._free.append(page)

    def refs(self, page: int) -> int:
        return self._refs[page]

    def shuffle_free(self, rng) -> None:
        """Reorders the free list (tests use it so that page ids do not follow positions)."""
        rng.shuffle(self._free)

    def check(self) -> None:
        """Invariant: free pages have no reference, held pages are not on the free list, nothing is lost."""
        free = set(self._free)
        assert len(free) == len(self._free), "a page is on the free list twice"
        for p in range(self.num_pages):
            assert (self._refs[p] == 0) == (p in free), f"page {p}: refs {self._refs[p]}, on free list {p in free}"
