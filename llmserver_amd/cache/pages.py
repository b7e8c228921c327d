"""Page allocator of one cache group: free list, reference counts, complete-page prefix hashes.

Semantics follow the reference's paged cache (/root/reference/utils/kv_cache.py:93-189):
pages come off the head of a FIFO free list; a page whose last reference goes away returns to
the tail of the free list, unless it holds a registered complete page of prompt tokens, in
which case it stays "idle" in least-recently-used order and can be shared again by digest; an
allocation that finds the free list empty evicts the oldest idle page, and fails with
:class:`CacheExhaustedError` only if there is none.
"""
from __future__ import annotations

from collections import OrderedDict, deque
from typing import List, Optional


class CacheExhaustedError(BufferError):
    """No page is free and none can be evicted (/root/reference/utils/kv_cache.py:516)."""


class CacheStateError(RuntimeError):
    """A page or slot is used in a way its state forbids (/root/reference/utils/kv_cache.py:519)."""


class PagePool:
    def __init__(self, num_pages: int, page_size: int):
        if num_pages <= 0:
            raise ValueError(f"num_pages must be positive: {num_pages}")
        if page_size <= 0:
            raise ValueError(f"page_size must be positive: {page_size}")
        self.num_pages, self.page_size = num_pages, page_size
        self.free_pages = deque(range(num_pages))
        self.references = [0] * num_pages
        self.allocated = set()
        self.cacheable = set()
        self.page_digest = {}
        self.digest_to_page = {}
        self.idle_lru: "OrderedDict[int, str]" = OrderedDict()

    # -- counts ------------------------------------------------------------------------
    @property
    def num_free(self) -> int:
        return len(self.free_pages)

    @property
    def num_idle(self) -> int:
        return len(self.idle_lru)

    @property
    def num_available(self) -> int:
        """Pages an allocation can get: free ones and idle cached ones (/root/reference/utils/engine.py:420)."""
        return len(self.free_pages) + len(self.idle_lru)

    def _check_id(self, page: int):
        if page < 0 or page >= self.num_pages:
            raise ValueError(f"Page id {page} is invalid, num_pages is {self.num_pages}")

    # -- allocate / retain / release -------------------------------------------------------
    def allocate(self) -> int:
        if not self.free_pages:
            if not self.idle_lru:
                raise CacheExhaustedError(f"Cache is out of pages: num_pages: {self.num_pages}, free: 0")
            self._discard(next(iter(self.idle_lru)))
        page = self.free_pages.popleft()
        self.allocated.add(page)
        self.references[page] = 1
        return page

    def retain(self, page: int) -> None:
        self._check_id(page)
        if page not in self.allocated:
            raise CacheStateError(f"Page {page} cannot be retained, it is not allocated")
        if self.references[page] == 0:
            self.idle_lru.pop(page, None)
        self.references[page] += 1

    def release(self, page: int) -> None:
        self._check_id(page)
        if page not in self.allocated:
            raise CacheStateError(f"Page {page} cannot be freed, it is not allocated")
        if self.references[page] == 0:
            raise CacheStateError(f"Page {page} cannot be freed, it has no active references")
        self.references[page] -= 1
        if self.references[page] > 0:
            return
        digest = self.page_digest.get(page)
        if page in self.cacheable and digest is not None and self.digest_to_page.get(digest) == page:
            self.idle_lru[page] = digest
            return
        self._discard(page)

    def _discard(self, page: int) -> None:
        self.idle_lru.pop(page, None)
        digest = self.page_digest.pop(page, None)
        if digest is not None and self.digest_to_page.get(digest) == page:
            del self.digest_to_page[digest]
        self.allocated.discard(page)
        self.cacheable.discard(page)
        self.free_pages.append(page)

    def release_table(self, table: List[int]) -> None:
        """Give back every page of a block table (entries < 0 were given back earlier); validates first."""
        seen = set()
        for page in table:
            if page < 0:
                continue
            if page not in self.allocated:
                raise CacheStateError(f"Page {page} cannot be freed, it is not allocated")
            if self.references[page] == 0:
                raise CacheStateError(f"Page {page} cannot be freed, it has no active references")
            if page in seen:
                raise ValueError(f"Duplicate page id {page} found")
            seen.add(page)
        for page in table:
            if page >= 0:
                self.release(page)
        table.clear()

    # -- prefix caching ------------------------------------------------------------------
    def register(self, page: int, digest: str) -> None:
        """Mark a complete page of prompt tokens shareable under ``digest``
        (/root/reference/utils/engine.py:387-401)."""
        if page not in self.allocated:
            raise CacheStateError(f"Page {page} cannot be cached, it isn't currently allocated")
        self.cacheable.add(page)
        self.page_digest[page] = digest
        self.digest_to_page.setdefault(digest, page)

    def find(self, digest: str) -> Optional[int]:
        page = self.digest_to_page.get(digest)
        if page is None or page not in self.allocated or page not in self.cacheable:
            return None
        if self.page_digest.get(page) != digest:
            return None
        return page

    def share(self, digest: str, table: List[int]) -> Optional[int]:
        """Append the page registered under ``digest`` to ``table`` and retain it
        (/root/reference/utils/kv_cache.py:124-135)."""
        page = self.find(digest)
        if page is None:
            return None
        if page in table:
            raise ValueError("One request must not list the same physical page twice")
        self.retain(page)
        table.append(page)
        return page

    def check_invariants(self) -> None:
        """Every page is in exactly one of: free list, idle, referenced."""
        free = list(self.free_pages)
        assert len(free) == len(set(free)), "a page is on the free list twice"
        for page in range(self.num_pages):
            states = (page in self.free_pages) + (page in self.idle_lru) + (self.references[page] > 0)
            assert states == 1, f"page {page} is in {states} states"
            assert (page in self.allocated) == (page not in self.free_pages)
