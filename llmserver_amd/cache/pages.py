"""The pages of one cache group and who has them.

Every page is in exactly one of three states.  FREE: nobody lists it and its content is worth nothing.  HELD: at
least one block table lists it (``holders`` counts the tables).  IDLE: nobody lists it, but it still holds a complete
page of prompt tokens that was published under a digest, so a later request with the same prefix can adopt it.
FREE and IDLE pages stand in two queues that are threaded through one pair of link arrays (a page is never in
both): new pages come from the front of the FREE queue and given-back pages join its end, so a page that was just
given back is the last to be written again; when no page is FREE the page that has been IDLE longest is recycled.

What the reference's paged cache does with a free deque, a set of allocated blocks, a set of cacheable blocks, two
digest maps and an ordered dict of idle blocks (utils/kv_cache.py:93-189) is one state and one digest per page here;
the outcomes its tests pin (order of reuse, eviction of the oldest idle block, errors on double frees) are the same.
"""
from __future__ import annotations

import enum
from typing import Dict, List, Optional


class CacheExhaustedError(BufferError):
    """No page is free and none can be recycled (utils/kv_cache.py:516 in the reference)."""


class CacheStateError(RuntimeError):
    """A page or slot is used in a way its state forbids (utils/kv_cache.py:519 in the reference)."""


class PageState(enum.IntEnum):
    FREE = 0
    IDLE = 1
    HELD = 2


class _Queue:
    """A first-in first-out queue of page numbers, linked through arrays it shares with its sibling."""

    def __init__(self, following: List[int], preceding: List[int]):
        self.following, self.preceding = following, preceding
        self.first = self.last = -1
        self.count = 0

    def join(self, page: int) -> None:
        self.following[page], self.preceding[page] = -1, self.last
        if self.last >= 0:
            self.following[self.last] = page
        else:
            self.first = page
        self.last = page
        self.count += 1

    def leave(self, page: int) -> None:
        before, after = self.preceding[page], self.following[page]
        if before >= 0:
            self.following[before] = after
        else:
            self.first = after
        if after >= 0:
            self.preceding[after] = before
        else:
            self.last = before
        self.following[page] = self.preceding[page] = -1
        self.count -= 1

    def __iter__(self):
        page = self.first
        while page >= 0:
            yield page
            page = self.following[page]


class PagePool:
    def __init__(self, num_pages: int, page_size: int):
        if num_pages <= 0 or page_size <= 0:
            raise ValueError(f"a pool needs a positive number of pages of a positive size, got {num_pages} pages of {page_size}")
        self.num_pages, self.page_size = num_pages, page_size
        self.state = [PageState.FREE] * num_pages
        self.holders = [0] * num_pages                         # block tables that list the page
        self.digest: List[Optional[str]] = [None] * num_pages  # what the page's tokens (and all before them) hash to, once complete
        self.by_digest: Dict[str, int] = {}                    # the one page that may be adopted under a digest
        following, preceding = [-1] * num_pages, [-1] * num_pages
        self._free, self._idle = _Queue(following, preceding), _Queue(following, preceding)
        for page in range(num_pages):
            self._free.join(page)

    # -- counts ----------------------------------------------------------------------------
    @property
    def num_free(self) -> int:
        return self._free.count

    @property
    def num_idle(self) -> int:
        return self._idle.count

    @property
    def num_available(self) -> int:
        """Pages that :meth:`allocate` can hand out: the free ones and the idle ones it may recycle."""
        return self._free.count + self._idle.count

    def _state_of(self, page: int) -> PageState:
        if not 0 <= page < self.num_pages:
            raise ValueError(f"there is no page {page} in a pool of {self.num_pages}")
        return self.state[page]

    def is_published(self, page: int) -> bool:
        digest = self.digest[page]
        return digest is not None and self.by_digest.get(digest) == page

    def published_pages(self) -> set:
        return set(self.by_digest.values())

    # -- taking and giving back --------------------------------------------------------------
    def _forget(self, page: int) -> None:
        digest, self.digest[page] = self.digest[page], None
        if digest is not None and self.by_digest.get(digest) == page:
            del self.by_digest[digest]

    def allocate(self) -> int:
        """A page for one block table to write into."""
        if self._free.count:
            page = self._free.first
            self._free.leave(page)
        elif self._idle.count:
            page = self._idle.first                  # idle longest: its cached tokens are given up
            self._idle.leave(page)
            self._forget(page)
        else:
            raise CacheExhaustedError(f"all {self.num_pages} pages of the pool are held")
        self.state[page], self.holders[page] = PageState.HELD, 1
        return page

    def hold(self, page: int) -> None:
        """One more block table lists ``page``."""
        state = self._state_of(page)
        if state == PageState.FREE:
            raise CacheStateError(f"page {page} is free: there is nothing on it to hold on to")
        if state == PageState.IDLE:
            self._idle.leave(page)
            self.state[page] = PageState.HELD
        self.holders[page] += 1

    def release(self, page: int) -> None:
        """One block table lists ``page`` no longer."""
        if self._state_of(page) != PageState.HELD:
            raise CacheStateError(f"page {page} is given back, but nobody holds it")
        self.holders[page] -= 1
        if self.holders[page]:
            return
        if self.is_published(page):
            self.state[page] = PageState.IDLE
            self._idle.join(page)
        else:
            self._forget(page)
            self.state[page] = PageState.FREE
            self._free.join(page)

    def release_all(self, table: List[int]) -> None:
        """Give back every page a block table lists (negative entries were given back earlier) and empty the table.
        Nothing is given back if any entry is wrong."""
        listed = [page for page in table if page >= 0]
        if len(set(listed)) != len(listed):
            raise ValueError(f"a block table lists a page twice: {sorted(listed)}")
        for page in listed:
            if self._state_of(page) != PageState.HELD:
                raise CacheStateError(f"page {page} is given back, but nobody holds it")
        for page in listed:
            self.release(page)
        table.clear()

    # -- complete pages of prompt tokens, shared by digest -------------------------------------------
    def publish(self, page: int, digest: str) -> None:
        """``page`` is complete; its tokens and everything before them hash to ``digest``.  The first page published
        under a digest is the one later requests adopt (utils/engine.py:387-401 in the reference)."""
        if self._state_of(page) != PageState.HELD:
            raise CacheStateError(f"page {page} cannot be published: nobody holds it")
        if self.digest[page] != digest:
            self._forget(page)
            self.digest[page] = digest
        self.by_digest.setdefault(digest, page)

    def lookup(self, digest: str) -> Optional[int]:
        page = self.by_digest.get(digest)
        if page is None or self.state[page] == PageState.FREE or self.digest[page] != digest:
            return None
        return page

    def adopt(self, digest: str, table: List[int], listed: Optional[set] = None) -> Optional[int]:
        """Append the page published under ``digest`` to ``table``; None if there is none.  ``listed``: the pages of
        ``table`` as a set, kept up to date here (who adopts many pages in a row passes it, so that the look whether
        the table has the page already does not walk the table each time)."""
        page = self.lookup(digest)
        if page is None:
            return None
        if page in (table if listed is None else listed):
            raise ValueError(f"page {page} is already in this block table")
        self.hold(page)
        table.append(page)
        if listed is not None:
            listed.add(page)
        return page

    # -- self-check ----------------------------------------------------------------------------
    def check_invariants(self) -> None:
        """Every page is in the one place its state names, and the digests point both ways."""
        queued = {PageState.FREE: list(self._free), PageState.IDLE: list(self._idle)}
        assert len(queued[PageState.FREE]) == self._free.count and len(queued[PageState.IDLE]) == self._idle.count, "a queue lost count"
        seen = queued[PageState.FREE] + queued[PageState.IDLE]
        assert len(seen) == len(set(seen)), "a page stands in a queue twice"
        for state, pages in queued.items():
            for page in pages:
                assert self.state[page] == state, f"page {page} stands in the {state.name} queue but is {self.state[page].name}"
        for page in range(self.num_pages):
            state = self.state[page]
            assert (self.holders[page] > 0) == (state == PageState.HELD), f"page {page} is {state.name} with {self.holders[page]} holders"
            if state != PageState.HELD:
                assert page in seen, f"page {page} is {state.name} but in no queue"
            if state == PageState.FREE:
                assert self.digest[page] is None, f"free page {page} still has a digest"
            if state == PageState.IDLE:
                assert self.is_published(page), f"idle page {page} is not published"
        for digest, page in self.by_digest.items():
            assert self.digest[page] == digest and self.state[page] != PageState.FREE, f"digest of page {page} points nowhere"
