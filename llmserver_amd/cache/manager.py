"""The cache manager: paged keys/values with a block table per request, and state slots.

Layers with the same cache needs form a group; every group has its own pages, its own allocator
and, per request, its own block table.  A group that keeps all keys frees a request's pages when
the request ends; a group with a window also frees a page as soon as every key on it has fallen
out of the window of all queries still to come.  Freed pages are used again.  Beside the pages
there are slots for per-request state of fixed size.

Page layout (one cache, i.e. one layer): keys ``[pages, kv_heads, page_size, head_dim]``, values
transposed ``[pages, kv_heads, head_dim, page_size]``, so that both attention products read each
lane's operand as one contiguous vector.  The reference keeps ``[layers, blocks, block_size,
kv_heads, head_dim]`` for both (utils/kv_cache.py:84-89 in the reference); the pages' states and
queues are in :mod:`.pages`.

Whoever plans a step asks this manager, never a block table, what the plan would cost: :meth:`pages_needed` and
:meth:`available_pages` answer per group, :meth:`token_room` says how far a request could grow on a given number
of pages in every group, :meth:`holds_anything` whether giving a request up would free anything.  A request's record
can be opened without a state slot (a request that waits computes nothing) and take one later (:meth:`acquire_state`).
"""
from __future__ import annotations

import dataclasses
import hashlib
from typing import Dict, List, Optional, Sequence

import numpy as np
import torch

from ..parts.base import PagedKVSpec, StateSpec
from .pages import CacheExhaustedError, CacheStateError, PagePool


@dataclasses.dataclass
class LayerCacheView:
    """What a mixer gets for one call of the order."""
    group: int
    keys: Optional[torch.Tensor]
    values: Optional[torch.Tensor]
    page_size: int
    writable: bool
    state: Optional[torch.Tensor] = None     # [slots, *shape] for a mixer with per-request state


SCRATCH_PAGES = 16      # fewest pages of storage beyond every pool (see CacheGroup.scratch_page)
SCRATCH_TOKENS = 512    # ... and as many as hold this many tokens: the filler tokens of a captured step with prompt portions


def scratch_pages(page_size: int) -> int:
    """Filler rows of one token take pages from the end of the scratch pages, a filler row of several tokens from their start."""
    return SCRATCH_PAGES + -(-SCRATCH_TOKENS // page_size)


class CacheGroup:
    def __init__(self, index: int, spec: PagedKVSpec, caches: List[int], num_pages: int, page_size: int):
        self.index, self.spec, self.caches = index, spec, caches
        self.pool = PagePool(num_pages, page_size)
        self.page_size = page_size
        self.scratch_pages = scratch_pages(page_size)
        self.keys = None     # [len(caches), pages + SCRATCH_PAGES, kv_heads, page_size, head_dim]
        self.values = None   # [len(caches), pages + SCRATCH_PAGES, kv_heads, head_dim, page_size]

    def scratch_page(self, index: int) -> int:
        """One of the pages behind the pool's, which no request ever holds: rows that a step adds to fill a captured
        shape write there (each filler row of one token its own page, a filler row of several tokens as many pages as
        it needs), and no request reads them."""
        if not 0 <= index < self.scratch_pages:
            raise ValueError(f"scratch pages are 0..{self.scratch_pages - 1}, asked for {index}")
        return self.pool.num_pages + index

    def first_needed_block(self, num_computed: int) -> int:
        """First logical block a query at position >= num_computed can still see."""
        if self.spec.window is None:
            return 0
        return max(0, num_computed - self.spec.window + 1) // self.page_size


class RequestCache:
    def __init__(self, request_id, n_groups: int):
        self.request_id = request_id
        self.tables: List[List[int]] = [[] for _ in range(n_groups)]
        self.state_slot = -1
        self.num_computed = 0
        self._arrays: List[Optional[np.ndarray]] = [None] * n_groups
        self._synced = [0] * n_groups       # entries of each table that its array mirrors

    def table_array(self, group: int) -> np.ndarray:
        """The group's block table as an int32 array (a view that the next call may overwrite).  A table mostly
        grows at its end, so only the new entries are converted; whoever changes entries in place or takes entries
        away calls :meth:`table_changed`."""
        table = self.tables[group]
        n, array, synced = len(table), self._arrays[group], min(self._synced[group], len(table))
        if array is None or array.shape[0] < n:
            grown = np.empty(max(64, 2 * n), dtype=np.int32)
            if synced:
                grown[:synced] = array[:synced]
            array = self._arrays[group] = grown
        if synced < n:
            array[synced:n] = table[synced:]
        self._synced[group] = n
        return array[:n]

    def table_changed(self, group: int) -> None:
        self._synced[group] = 0


class CacheManager:
    def __init__(self, cache_specs: Dict[int, object], page_size: int, num_pages, num_state_slots: int = 0,
                 device=None, dtype=torch.float32, allocate_storage: bool = True, model_identity: str = "model"):
        self.page_size = page_size
        self.device, self.dtype = device, dtype
        self.model_identity = model_identity
        self._identity_bytes = str(model_identity).encode("utf-8")
        self.groups: List[CacheGroup] = []
        self.group_of_cache: Dict[int, int] = {}
        self.layer_in_group: Dict[int, int] = {}
        self.state_specs: Dict[int, StateSpec] = {}
        by_spec: Dict[PagedKVSpec, List[int]] = {}
        for cache, spec in sorted(cache_specs.items()):
            if isinstance(spec, PagedKVSpec):
                by_spec.setdefault(spec, []).append(cache)
            elif isinstance(spec, StateSpec):
                self.state_specs[cache] = spec
            else:
                raise TypeError(f"cache {cache}: unknown cache spec {spec!r}")
        for spec, caches in by_spec.items():
            pages = num_pages[len(self.groups)] if isinstance(num_pages, (list, tuple)) else num_pages
            group = CacheGroup(len(self.groups), spec, caches, pages, page_size)
            for position, cache in enumerate(caches):
                self.group_of_cache[cache] = group.index
                self.layer_in_group[cache] = position
            self.groups.append(group)
        self.num_state_slots = num_state_slots if self.state_specs else 0
        self.free_state_slots = list(range(self.num_state_slots - 1, -1, -1))
        self.state: Dict[int, torch.Tensor] = {}
        self.requests: Dict[object, RequestCache] = {}
        self.prefix_caching_possible = bool(self.groups) and not self.state_specs and all(
            group.spec.window is None for group in self.groups)
        if allocate_storage:
            self._allocate_storage()

    def _allocate_storage(self):
        for group in self.groups:
            spec, n = group.spec, len(group.caches)
            pages = group.pool.num_pages + group.scratch_pages
            group.keys = torch.zeros((n, pages, spec.n_kv_heads, self.page_size, spec.head_dim), device=self.device, dtype=self.dtype)
            group.values = torch.zeros((n, pages, spec.n_kv_heads, spec.head_dim, self.page_size), device=self.device, dtype=self.dtype)
        for cache, spec in self.state_specs.items():
            self.state[cache] = torch.zeros((max(1, self.num_state_slots), *spec.shape), device=self.device,
                                            dtype=getattr(torch, spec.dtype))

    @staticmethod
    def bytes_per_token(cache_specs: Dict[int, object], dtype: torch.dtype) -> int:
        size = torch.empty(0, dtype=dtype).element_size()
        return sum(2 * spec.n_kv_heads * spec.head_dim * size for spec in cache_specs.values() if isinstance(spec, PagedKVSpec))

    # -- views for the model ---------------------------------------------------------------
    def view(self, call) -> LayerCacheView:
        cache = call.cache
        if cache in self.group_of_cache:
            group = self.groups[self.group_of_cache[cache]]
            layer = self.layer_in_group[cache]
            return LayerCacheView(group.index, None if group.keys is None else group.keys[layer],
                                  None if group.values is None else group.values[layer], self.page_size, call.writes_cache)
        if cache in self.state:
            return LayerCacheView(-1, None, None, self.page_size, call.writes_cache, self.state[cache])
        return LayerCacheView(-1, None, None, self.page_size, call.writes_cache)

    # -- requests ------------------------------------------------------------------------
    def open(self, request_id, state: bool = True) -> RequestCache:
        """A record for a new request: empty block tables and, unless ``state`` is False, a state slot (if any mixer
        keeps state).  Nothing is opened if no slot is free."""
        if request_id in self.requests:
            raise CacheStateError(f"request {request_id!r} already has a cache")
        record = RequestCache(request_id, len(self.groups))
        if state:
            self._take_slot(record)
        self.requests[request_id] = record
        return record

    def _take_slot(self, record: RequestCache) -> None:
        if not self.state_specs or record.state_slot >= 0:
            return
        if not self.free_state_slots:
            raise CacheExhaustedError(f"all {self.num_state_slots} state slots are taken")
        record.state_slot = self.free_state_slots.pop()
        for tensor in self.state.values():
            tensor[record.state_slot].zero_()            # a state starts from nothing

    def acquire_state(self, request_id) -> int:
        """The request is about to compute: give it a state slot (zeroed) if mixers keep state and it has none yet.
        Returns the slot, -1 for a model without state."""
        record = self.record(request_id)
        self._take_slot(record)
        return record.state_slot

    def state_slots_free(self) -> Optional[int]:
        """How many more requests can get a state slot; None if no mixer keeps state (then nothing limits them)."""
        return len(self.free_state_slots) if self.state_specs else None

    def has(self, request_id) -> bool:
        return request_id in self.requests

    def record(self, request_id) -> RequestCache:
        if request_id not in self.requests:
            raise KeyError(f"Request does not have a cache: {request_id!r}")
        return self.requests[request_id]

    def pages_needed(self, request_id, num_tokens: int) -> List[int]:
        """Pages each group must still allocate so that positions < num_tokens are covered."""
        record = self.requests.get(request_id)
        needed = []
        for group in self.groups:
            have = len(record.tables[group.index]) if record is not None else 0
            needed.append(max(0, -(-num_tokens // self.page_size) - have))
        return needed

    def available_pages(self) -> List[int]:
        return [group.pool.num_available for group in self.groups]

    def token_room(self, request_id, spare_pages: Sequence[int]) -> int:
        """The number of leading positions of the request that its pages would cover if every group gave it
        ``spare_pages[group]`` more (what it holds already counts).  Without paged groups nothing bounds it."""
        record = self.requests.get(request_id)
        room = None
        for group in self.groups:
            have = len(record.tables[group.index]) if record is not None else 0
            covered = (have + max(0, int(spare_pages[group.index]))) * self.page_size
            room = covered if room is None else min(room, covered)
        return (1 << 62) if room is None else room

    def holds_anything(self, request_id) -> bool:
        """Whether closing the request's record would give anything back: a page in any group, or a state slot."""
        record = self.requests.get(request_id)
        if record is None:
            return False
        return record.state_slot >= 0 or any(page >= 0 for table in record.tables for page in table)

    def ensure(self, request_id, num_tokens: int) -> None:
        """Allocate pages so that positions ``< num_tokens`` have a place in every group.

        All-or-nothing: if any group runs out, pages taken by this call are given back and
        :class:`CacheExhaustedError` is raised.
        """
        record = self.record(request_id)
        taken = []
        try:
            for group in self.groups:
                table = record.tables[group.index]
                wanted = -(-num_tokens // self.page_size)
                while len(table) < wanted:
                    page = group.pool.allocate()
                    table.append(page)
                    taken.append((group, page))
        except CacheExhaustedError:
            for group, page in reversed(taken):
                table = record.tables[group.index]
                assert table[-1] == page
                table.pop()
                record.table_changed(group.index)
                group.pool.release(page)
            raise

    def advance(self, request_id, num_computed: int) -> None:
        """Tokens ``< num_computed`` are in the cache; give back pages a window has passed."""
        record = self.record(request_id)
        record.num_computed = num_computed
        for group in self.groups:
            if group.spec.window is None:
                continue
            table = record.tables[group.index]
            for block in range(min(group.first_needed_block(num_computed), len(table))):
                if table[block] >= 0:
                    group.pool.release(table[block])
                    table[block] = -1
                    record.table_changed(group.index)

    def close(self, request_id) -> None:
        """The request ended (or is preempted): everything it holds is given back."""
        record = self.record(request_id)
        for group in self.groups:
            group.pool.release_all(record.tables[group.index])
        if record.state_slot >= 0:
            self.free_state_slots.append(record.state_slot)
            record.state_slot = -1
        del self.requests[request_id]

    # -- prefix caching (complete pages of prompt tokens) ------------------------------------
    def digest(self, parent: str, tokens: Sequence[int]) -> str:
        """Chained sha256 over (parent digest, page tokens, model, adapter), root parent "root"
        (utils/engine.py:193-195)."""
        return self._digest(parent, np.asarray(tokens, dtype=np.int64).tobytes())

    def _digest(self, parent: str, page_tokens: bytes) -> str:
        # (the tokens as 64-bit integers, the rest as text; the lengths of the parts are fixed or delimited, so no two
        # different inputs give the same bytes)
        return hashlib.sha256(b"%s|%d|%s|%s|none" % (parent.encode("ascii"), len(page_tokens), page_tokens, self._identity_bytes)).hexdigest()

    def prefix_digests(self, prompt: Sequence[int]) -> List[str]:
        """The chained digests of the prompt's complete pages that may be shared (at least one
        prompt token always remains to be computed)."""
        digests, parent = [], "root"
        blocks = (len(prompt) - 1) // self.page_size
        data = np.asarray(prompt[:blocks * self.page_size], dtype=np.int64).tobytes()       # converted once, not page by page
        page_bytes = 8 * self.page_size
        for block in range(blocks):
            parent = self._digest(parent, data[block * page_bytes:(block + 1) * page_bytes])
            digests.append(parent)
        return digests

    def share_prefix(self, request_id, prompt: Sequence[int], digests: Optional[List[str]] = None) -> int:
        """Attach the longest chain of cached complete pages; always leaves at least one prompt
        token to compute (utils/engine.py:197-208).  May be called again while
        the request has computed nothing itself: the chain is then continued.  Returns the
        tokens newly covered."""
        if not self.prefix_caching_possible:
            return 0
        record = self.record(request_id)
        have = len(record.tables[0])
        if any(len(record.tables[group.index]) != have for group in self.groups) or record.num_computed != have * self.page_size:
            raise CacheStateError("a prefix can only be shared into a block table that holds shared pages only")
        if digests is None:
            digests = self.prefix_digests(prompt)
        covered = 0
        listed = [set(record.tables[group.index]) for group in self.groups]      # (a table never lists a page twice)
        for digest in digests[have:]:
            if any(group.pool.lookup(digest) is None for group in self.groups):
                break
            for group in self.groups:
                group.pool.adopt(digest, record.tables[group.index], listed[group.index])
            covered += self.page_size
        record.num_computed += covered
        return covered

    def register_prefix(self, request_id, prompt: Sequence[int], old_computed: int, new_computed: int) -> None:
        """Register pages of prompt tokens that became complete between two counts of computed
        tokens (utils/engine.py:383-401)."""
        if not self.prefix_caching_possible:
            return
        record = self.record(request_id)
        old_complete = min(old_computed, len(prompt)) // self.page_size
        new_complete = min(new_computed, len(prompt)) // self.page_size
        for block in range(old_complete, new_complete):
            tokens = prompt[block * self.page_size:(block + 1) * self.page_size]
            for group in self.groups:
                table = record.tables[group.index]
                parent = "root" if block == 0 else group.pool.digest[table[block - 1]]
                group.pool.publish(table[block], self.digest(parent, tokens))

    def check_invariants(self) -> None:
        for group in self.groups:
            group.pool.check_invariants()
            held = {}
            for record in self.requests.values():
                for page in record.tables[group.index]:
                    if page >= 0:
                        held[page] = held.get(page, 0) + 1
            for page in range(group.pool.num_pages):
                assert group.pool.holders[page] == held.get(page, 0), (
                    f"group {group.index} page {page}: the pool counts {group.pool.holders[page]} holders, {held.get(page, 0)} tables list it")
        slots = [record.state_slot for record in self.requests.values() if record.state_slot >= 0]
        assert len(slots) == len(set(slots)), "a state slot is held twice"
        assert not set(slots) & set(self.free_state_slots), "a held state slot is on the free list"
        if self.state_specs:
            assert len(slots) + len(self.free_state_slots) == self.num_state_slots, "a state slot was lost"
