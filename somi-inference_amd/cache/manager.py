"""The cache manager: paged keys/values per group of layers, block tables per request,
and slots for fixed-size per-request state.

Reference: ``KVCacheManager`` (somi_inference/core/paged_attention.py:112-296):
one allocator, one tensor per layer, per-sequence page lists and token counts;
``allocate_slots`` before the forward and ``advance_tokens`` after it
(:202-221, :294-296); ``free_sequence`` returns every page (:195-200); a
duplicate ``register_sequence`` raises "already registered" (:150-156).

Beyond the reference: a layer says what it keeps per token (a ``PagedSpec``: the
tensors of a page, a window, a page size of its own if its kernels want one) and
layers are put into *groups* by window and page size.  The layers of a group
share one page pool and one block table per request; each has tensors of its own,
allocated as its spec lists them.  A group with a window releases a page as soon
as the window has passed it, while the request is still live.  Every group's pool
holds the same number of tokens, ``num_blocks * block_size``, cut into pages of
the group's size.  Mixers with fixed-size state get one slot per request in a
state tensor (this architecture has none; the slot is assigned all the same so
nothing changes when one is added).
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Hashable

import numpy as np
import torch

from ..parts.base import FixedStateSpec, LayerCache, PagedSpec
from .pool import CacheError, OutOfPages, PagePool

RELEASED = -1     # host-side mark of a logical page a window has passed


@dataclass
class PagedGroup:
    window: int | None
    pool: PagePool
    page_size: int = 0
    runs: list[int] = field(default_factory=list)      # layer runs whose tensors use this group's page ids


@dataclass
class RequestCache:
    num_tokens: int = 0
    pages: list[list[int]] = field(default_factory=list)   # per group: logical page -> physical page or RELEASED
    state_slot: int = -1
    # per group: the same as ``pages`` as an int32 array for the kernels' block tables (released pages read
    # as page 0: the kernels never look below a window); kept beside the lists so that laying out a step
    # copies a slice instead of walking every page of every request
    rows: list[np.ndarray] = field(default_factory=list)

    def note_page(self, group: int, logical: int, page: int) -> None:
        row = self.rows[group]
        if logical >= row.size:
            grown = np.zeros(max(16, 2 * row.size, logical + 1), dtype=np.int32)
            grown[:row.size] = row
            self.rows[group] = row = grown
        row[logical] = page


class CacheManager:
    def __init__(self, needs: list[PagedSpec | FixedStateSpec | int | None], *, block_size: int,
                 num_blocks: int, max_requests: int, dtype: torch.dtype, device: torch.device | str,
                 allocate_tensors: bool = True) -> None:
        """``block_size``: tokens per page where a spec names no page size of its own.  ``num_blocks``: pages of
        that size per group; a group with another page size gets as many pages as hold the same tokens."""
        if block_size < 1 or num_blocks < 1 or max_requests < 1:
            raise ValueError("block_size, num_blocks and max_requests must be >= 1")
        self.block_size, self.num_blocks, self.max_requests = int(block_size), int(num_blocks), int(max_requests)
        self.dtype, self.device = dtype, torch.device(device)
        self.groups: list[PagedGroup] = []
        self.layer_caches: list[LayerCache | None] = [None] * len(needs)
        by_need: dict[tuple[int | None, int], int] = {}
        for run, need in enumerate(needs):
            if isinstance(need, PagedSpec):
                page_size = int(need.page_size or self.block_size)
                key = (need.window, page_size)
                if key not in by_need:
                    pages = self.pool_tokens // page_size
                    if pages < 1:
                        raise ValueError(f"a pool of {self.pool_tokens} tokens holds no page of {page_size}")
                    by_need[key] = len(self.groups)
                    self.groups.append(PagedGroup(need.window, PagePool(pages), page_size))
                group = by_need[key]
                self.groups[group].runs.append(run)
                tensors = {}
                if allocate_tensors:
                    pages = self.groups[group].pool.num_pages
                    tensors = {t.name: torch.zeros((pages, *t.page_shape(page_size)), dtype=t.dtype or dtype,
                                                   device=self.device) for t in need.tensors}
                self.layer_caches[run] = LayerCache(need, group, tensors=tensors, page_size=page_size)
            elif isinstance(need, FixedStateSpec):
                state = None
                if allocate_tensors:
                    # one row more than there are requests: the slot that padding entries of a step use
                    state = torch.zeros((self.max_requests + 1, *need.shape), dtype=need.dtype, device=self.device)
                self.layer_caches[run] = LayerCache(need, -1, state=state)
        for run, need in enumerate(needs):          # runs that read an earlier run's cache
            if isinstance(need, int) and not isinstance(need, bool):
                source = self.layer_caches[need]
                if source is None:
                    raise CacheError(f"run {run} reads the cache of run {need}, which has none")
                self.layer_caches[run] = LayerCache(source.spec, source.group, tensors=source.tensors,
                                                    state=source.state, writes=False, page_size=source.page_size)
        self._requests: dict[Hashable, RequestCache] = {}
        self._free_slots = list(range(self.max_requests - 1, -1, -1))
        self.padding_state_slot = self.max_requests       # never handed to a request

    @property
    def pool_tokens(self) -> int:
        """Tokens that each group's pool holds."""
        return self.num_blocks * self.block_size

    @staticmethod
    def page_bytes(needs: list, block_size: int, dtype: torch.dtype) -> int:
        """Bytes of device memory that ``block_size`` more tokens per group cost: every tensor of every run that
        writes (a group with pages of another size holds the same tokens in other pages)."""
        def item(kind: torch.dtype | None) -> int:
            return torch.empty((), dtype=kind or dtype).element_size()
        return sum(t.elements_per_token() * int(block_size) * item(t.dtype)
                   for need in needs if isinstance(need, PagedSpec) for t in need.tensors)

    # --------------------------------------------------------------- requests
    def has(self, request_id: Hashable) -> bool:
        return request_id in self._requests

    def live_requests(self) -> list[Hashable]:
        return list(self._requests)

    def register(self, request_id: Hashable) -> None:
        if request_id in self._requests:
            raise CacheError(f"request {request_id!r} is already registered")
        if not self._free_slots:
            raise CacheError(f"all {self.max_requests} request slots are in use")
        slot = self._free_slots.pop()
        self._requests[request_id] = RequestCache(0, [[] for _ in self.groups], slot,
                                                  [np.zeros(16, dtype=np.int32) for _ in self.groups])
        for cache in self.layer_caches:
            if cache is not None and cache.state is not None and cache.writes:
                cache.state[slot].zero_()

    def free(self, request_id: Hashable) -> None:
        """Give back every page and the state slot of a request."""
        record = self._get(request_id)
        for group, pages in zip(self.groups, record.pages):
            for page in pages:
                if page != RELEASED:
                    group.pool.release(page)
        self._free_slots.append(record.state_slot)
        del self._requests[request_id]

    def _get(self, request_id: Hashable) -> RequestCache:
        if request_id not in self._requests:
            raise CacheError(f"request {request_id!r} is not registered")
        return self._requests[request_id]

    def num_tokens(self, request_id: Hashable) -> int:
        return self._get(request_id).num_tokens

    def state_slot(self, request_id: Hashable) -> int:
        return self._get(request_id).state_slot

    # ------------------------------------------------------------------ pages
    def _pages_for(self, group: PagedGroup, length: int) -> int:
        return (length + group.page_size - 1) // group.page_size

    def holds(self, tokens: int) -> bool:
        """Whether a request of this many tokens fits the pools when it runs alone."""
        return all(self._pages_for(group, tokens) <= group.pool.num_pages for group in self.groups)

    def pages_needed(self, request_id: Hashable, new_tokens: int) -> list[int]:
        """Per group, how many pages a portion of ``new_tokens`` more tokens has to take."""
        record = self._get(request_id)
        return [max(0, self._pages_for(group, record.num_tokens + new_tokens) - len(pages))
                for group, pages in zip(self.groups, record.pages)]

    def tokens_within(self, request_id: Hashable, free: list[int]) -> int:
        """How many more tokens the request can hold if group g may take ``free[g]`` more pages."""
        record = self._get(request_id)
        room = min(((len(pages) + spare) * group.page_size
                    for group, pages, spare in zip(self.groups, record.pages, free)), default=None)
        return max(0, room - record.num_tokens) if room is not None else 1 << 62

    def free_pages(self) -> list[int]:
        return [group.pool.num_free for group in self.groups]

    def can_reserve(self, portions: list[tuple[Hashable, int]]) -> bool:
        want = [0] * len(self.groups)
        for request_id, new_tokens in portions:
            for g, n in enumerate(self.pages_needed(request_id, new_tokens)):
                want[g] += n
        return all(w <= f for w, f in zip(want, self.free_pages()))

    def reserve(self, request_id: Hashable, new_tokens: int) -> None:
        """Take the pages that positions ``num_tokens .. num_tokens + new_tokens - 1`` fall in.

        Either every group gets its pages or nothing changes (then :class:`OutOfPages`).
        """
        if new_tokens < 1:
            raise CacheError("a portion holds at least one token")
        record = self._get(request_id)
        needed = self.pages_needed(request_id, new_tokens)
        for group, n in zip(self.groups, needed):
            if n > group.pool.num_free:
                raise OutOfPages(f"request {request_id!r} needs {n} more pages, {group.pool.num_free} are free")
        for g, (group, pages, n) in enumerate(zip(self.groups, record.pages, needed)):
            for _ in range(n):
                pages.append(group.pool.allocate())
                record.note_page(g, len(pages) - 1, pages[-1])

    def rollback(self, request_id: Hashable) -> None:
        """Give back the pages that were reserved beyond the committed tokens (a step that failed after
        ``reserve`` and before ``commit``); what the committed tokens hold stays."""
        record = self._get(request_id)
        for group, pages in zip(self.groups, record.pages):
            keep = self._pages_for(group, record.num_tokens)
            while len(pages) > keep:
                page = pages.pop()
                if page != RELEASED:
                    group.pool.release(page)

    def commit(self, request_id: Hashable, new_tokens: int) -> None:
        """Count the tokens a step wrote, and give back pages a window has passed."""
        record = self._get(request_id)
        record.num_tokens += new_tokens
        for g, (group, pages) in enumerate(zip(self.groups, record.pages)):
            if self._pages_for(group, record.num_tokens) > len(pages):
                raise CacheError(f"request {request_id!r}: tokens committed beyond the reserved pages")
            if group.window is None:
                continue
            # The next token sits at position num_tokens and sees keys from
            # num_tokens - window + 1 on; pages wholly below that are done.
            first_visible = record.num_tokens - group.window + 1
            for logical in range(min(len(pages), max(0, first_visible) // group.page_size)):
                if pages[logical] != RELEASED:
                    group.pool.release(pages[logical])
                    pages[logical] = RELEASED
                    record.note_page(g, logical, 0)

    # ------------------------------------------------------- tables for a step
    def page_list(self, group: int, request_id: Hashable) -> list[int]:
        return self._get(request_id).pages[group]

    def table_row(self, group: int, request_id: Hashable) -> np.ndarray:
        """The request's block-table row for the kernels: int32, one entry per logical page, released pages as 0."""
        record = self._get(request_id)
        return record.rows[group][:len(record.pages[group])]

    def slots(self, group: int, request_id: Hashable, start: int, count: int) -> list[int]:
        """Physical slot (page * page size + offset) of positions start .. start + count - 1."""
        pages = self._get(request_id).pages[group]
        size = self.groups[group].page_size
        out = []
        for pos in range(start, start + count):
            page = pages[pos // size]
            if page == RELEASED:
                raise CacheError(f"position {pos} of request {request_id!r} lies in a released page")
            out.append(page * size + pos % size)
        return out

    # -------------------------------------------------------------- invariants
    def check_invariants(self) -> None:
        """No page lost, held twice or free while held; slots likewise."""
        for g, group in enumerate(self.groups):
            held: dict[int, Hashable] = {}
            for request_id, record in self._requests.items():
                for page in record.pages[g]:
                    if page == RELEASED:
                        continue
                    if page in held:
                        raise CacheError(f"group {g}: page {page} held by {held[page]!r} and {request_id!r}")
                    held[page] = request_id
            for request_id, record in self._requests.items():
                mirror = [0 if page == RELEASED else page for page in record.pages[g]]
                if record.rows[g][:len(mirror)].tolist() != mirror:
                    raise CacheError(f"group {g}: the block-table row of {request_id!r} differs from its pages")
            free = group.pool.free_pages()
            if len(set(free)) != len(free):
                raise CacheError(f"group {g}: a page is on the free list twice")
            if set(free) & set(held):
                raise CacheError(f"group {g}: pages both free and held: {sorted(set(free) & set(held))}")
            if len(free) + len(held) != group.pool.num_pages:
                raise CacheError(f"group {g}: {group.pool.num_pages - len(free) - len(held)} pages lost")
            for page in held:
                if group.pool.refcount(page) != 1:
                    raise CacheError(f"group {g}: page {page} has refcount {group.pool.refcount(page)}")
        slots = [r.state_slot for r in self._requests.values()]
        if len(set(slots)) != len(slots) or set(slots) & set(self._free_slots):
            raise CacheError("a state slot is held twice or both free and held")
        if len(slots) + len(self._free_slots) != self.max_requests:
            raise CacheError("a state slot is lost")
