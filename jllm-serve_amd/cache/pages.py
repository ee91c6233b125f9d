"""A pool of page ids: free list and reference counts, nothing else. The pool itself is native code
(csrc/host/host_core.cpp); this class is its face.

The reference's pool hands out block ids from a free list, counts references and raises when every
block is referenced (kv/KvPool.java:249-302, kv/KvPoolExhausted.java:4-8). The prefix tree and the eviction of
cached pages live beside this class (cache/prefix.py, driven by the cache manager); the spill tiers of the
reference's pool are not part of this engine. The contract kept here is: a page is either free or
held, ``alloc`` never returns a held page, ``release`` of the last reference makes it free at once.
"""
from __future__ import annotations

import ctypes

import numpy as np

from .. import host


class OutOfPages(RuntimeError):
    """No free page (kv/KvPoolExhausted.java). The scheduler decides what happens next."""


class PagePool:
    def __init__(self, num_pages: int, page_tokens: int):
        if num_pages < 1 or page_tokens < 1:
            raise ValueError(f"a pool needs at least one page of at least one token, got {num_pages} x {page_tokens}")
        self.num_pages = num_pages
        self.page_tokens = page_tokens
        self._lib = host.library()
        self._pool = ctypes.c_void_p(self._lib.jllm_pool_new(num_pages))
        if not self._pool:
            raise MemoryError(f"no pool of {num_pages} pages")

    def __del__(self):
        pool, self._pool = getattr(self, "_pool", None), None
        if pool:
            try:
                self._lib.jllm_pool_delete(pool)
            except Exception:  # the interpreter is shutting down and the library is gone: so is its memory
                pass

    @property
    def free_pages(self) -> int:
        return self._lib.jllm_pool_free_pages(self._pool)

    @property
    def used_pages(self) -> int:
        return self.num_pages - self.free_pages

    @property
    def high_water(self) -> int:
        return self._lib.jllm_pool_high_water(self._pool)

    @property
    def allocations(self) -> int:
        return self._lib.jllm_pool_allocations(self._pool)

    def alloc(self) -> int:
        p = self._lib.jllm_pool_alloc(self._pool)
        if p < 0:
            raise OutOfPages(f"the KV pool is full: all {self.num_pages} pages of {self.page_tokens} positions are "
                             "in use by running sequences")
        return p

    def retain(self, page: int) -> None:
        if self._lib.jllm_pool_retain(self._pool, int(page)) < 0:
            raise ValueError(f"page {page} is not held")

    def release(self, page: int) -> None:
        if self._lib.jllm_pool_release(self._pool, int(page)) < 0:
            raise ValueError(f"page {page} released but not held")

    def refs(self, page: int) -> int:
        r = self._lib.jllm_pool_refs(self._pool, int(page))
        if r < 0:
            raise IndexError(f"the pool has no page {page}")
        return r

    def free_list(self) -> list:
        """The free pages; the last one is handed out next."""
        buf = np.empty(max(1, self.num_pages), np.int32)
        n = self._lib.jllm_pool_free_list(self._pool, buf.ctypes.data)
        return buf[:n].tolist()

    def shuffle_free(self, rng) -> None:
        """Reorders the free list (tests use it so that page ids do not follow positions)."""
        order = self.free_list()
        rng.shuffle(order)
        arr = np.asarray(order, np.int32)
        if self._lib.jllm_pool_set_free_list(self._pool, arr.ctypes.data, len(order)) != 0:
            raise AssertionError("the shuffled list does not hold the free pages")

    def check(self) -> None:
        """Invariant: free pages have no reference, held pages are not on the free list, nothing is lost."""
        page = ctypes.c_int(-1)
        rc = self._lib.jllm_pool_check(self._pool, ctypes.byref(page))
        assert rc != 1, f"page {page.value} is on the free list twice"
        assert rc != 2, f"page {page.value}: refs {self.refs(page.value)}, and the free list says otherwise"
