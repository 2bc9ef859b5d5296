"""The cache manager: pages with a block table per request, and state slots.

Run entries of the model declare what they need (``cache.needs``): something in pages
(keys and values, ``PagedKVNeed``, perhaps with a window; or whatever payload a need's class
allocates) or per-request state of fixed size (``StateNeed``). Entries with equal paged needs form a
group; a group has a pool of its own, every entry its own page arrays (keys and values lie in tiles of
16 positions, see ``cache.layout``), and every request has one block table per group. Pages are taken when
a request's tokens cross a page's edge, given back when the request is closed,
and, in a group with a window, as soon as every position on them is older than
any later query can see. Nothing is cleared on reuse: lengths, not contents,
say what is valid. The reference has no pages: one ``[slots, kv_heads, capacity,
head_dim]`` tensor per layer, zero-filled on release (src/inference/kv_cache.cpp:11-64).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, Hashable, List, Optional, Sequence

import numpy as np
import torch

from .needs import Binding, CacheNeed, PagedBinding, PagedKVNeed, StateBinding, StateNeed
from .pages import OutOfPages, PagePool, SlotPool

RELEASED = -1  # block-table entry of a page that a window has passed


@dataclass
class RequestCache:
    request_id: Hashable
    slot: int
    num_tokens: int = 0                      # positions whose keys, values and state are in the cache
    reserved: int = 0                        # positions beyond num_tokens that already have pages
    pages: List[List[int]] = field(default_factory=list)  # per group: page of every block, RELEASED if given back
    closed: bool = False
    broken: bool = False                     # its state may hold part of a step that failed: only closing is left


class CacheGroup:
    def __init__(self, index: int, need: CacheNeed, num_pages: int, page_size: int, max_requests: int,
                 max_blocks: int):
        self.index = index
        self.need = need
        self.page_size = page_size
        self.pool = PagePool(num_pages)
        self.entries: List[int] = []
        # The block tables of all live requests, one row per state slot, kept up to date as pages come and go:
        # a step gathers its rows from here instead of rebuilding them from lists.
        self.tables = np.full((max_requests, max_blocks), RELEASED, dtype=np.int32)

    def first_needed_block(self, num_tokens: int) -> int:
        """Blocks below this index hold no key that a query at ``num_tokens`` or later can see."""
        if self.need.window is None:
            return 0
        oldest_visible = num_tokens - self.need.window + 1
        return max(0, oldest_visible) // self.page_size


def window_blocks(window: int, portion: int, page_size: int) -> int:
    """The most blocks a request holds in a group with this window while steps bring it at most ``portion``
    tokens: the blocks between the oldest key that the portion's first query sees and its last token."""
    return -(-(window - 1 + portion) // page_size) + 1


def pages_of_group(need: CacheNeed, num_pages: int, page_size: int, max_requests: int,
                   max_portion: Optional[int]) -> int:
    """How many pages a group's pool gets of the ``num_pages`` asked for: all of them, unless the group has a
    window and the largest portion of a step is known; then no more than every request slot can hold at once."""
    if need.window is None or max_portion is None:
        return num_pages
    return max(1, min(num_pages, max_requests * window_blocks(need.window, max_portion, page_size)))


class CacheManager:
    def __init__(self, needs: Sequence[CacheNeed], reads: Sequence[Optional[int]], page_size: int,
                 num_pages: int, max_requests: int, dtype: torch.dtype = torch.float32,
                 device: Optional[torch.device] = None, max_blocks: Optional[int] = None,
                 max_portion: Optional[int] = None):
        """``num_pages``: the pages of a group that keeps every key. A group with a window gets fewer if
        ``max_portion`` says how many tokens a step brings a request at most (``pages_of_group``): a model of
        mostly windowed layers then does not pay for the full pool in every group. ``max_blocks``: the most
        blocks a request's table has (its positions / page size); by default the pool's size."""
        if page_size <= 0:
            raise ValueError("page_size must be positive")
        if len(needs) != len(reads):
            raise ValueError("one need and one read source per run entry")
        self.page_size = page_size
        self.max_requests = max_requests
        self.max_blocks = max_blocks if max_blocks else num_pages   # most blocks a request's table has (a window gives early ones back)
        self.max_portion = max_portion
        self.dtype = dtype
        self.device = device
        self.groups: List[CacheGroup] = []
        self.slots = SlotPool(max_requests)
        self.requests: Dict[Hashable, RequestCache] = {}
        self._bindings: List[Optional[Binding]] = [None] * len(needs)
        self._slot_storage: List[tuple] = []        # (need, storage) of every run entry that keeps state in slots
        by_need: Dict[CacheNeed, CacheGroup] = {}
        for entry, need in enumerate(needs):
            if reads[entry] is not None or need is None:
                continue
            if not isinstance(need, CacheNeed):
                raise TypeError(f"run entry {entry} declares an unknown cache need {need!r}")
            if need.paged:
                if device is not None:
                    need.check_page_size(page_size)   # the layout on the device may ask more of a page than the books do
                group = by_need.get(need)
                if group is None:
                    group = CacheGroup(len(self.groups), need, pages_of_group(need, num_pages, page_size, max_requests, max_portion),
                                       page_size, max_requests, self.max_blocks)
                    self.groups.append(group)
                    by_need[need] = group
                group.entries.append(entry)
                storage = need.allocate_pages(group.pool.num_pages, page_size, dtype, device) if device is not None else None
                self._bindings[entry] = need.bind(group.index, storage, True)
            else:
                storage = need.allocate_slots(max_requests, dtype, device) if device is not None else None
                if storage is not None:
                    self._slot_storage.append((need, storage))
                self._bindings[entry] = need.bind(None, storage, True)
        for entry, source in enumerate(reads):
            if source is None:
                continue
            binding = self._bindings[source]
            if binding is None:
                raise ValueError(f"run entry {entry} reads the cache of entry {source}, which has none")
            self._bindings[entry] = binding.shared()

    # ---- what the model sees -------------------------------------------------------------
    @property
    def has_state(self) -> bool:
        """Whether any run entry keeps per-request state of fixed size (which, unlike pages, a failed step cannot
        simply leave behind)."""
        return any(binding is not None and not binding.need.paged and binding.owned for binding in self._bindings)

    def bindings(self) -> List[object]:
        return list(self._bindings)

    # ---- requests ------------------------------------------------------------------------
    def open(self, request_id: Hashable) -> RequestCache:
        if request_id in self.requests:
            raise KeyError(f"request {request_id!r} is already open")
        slot = self.slots.take_one()
        for need, storage in self._slot_storage:
            need.zero_slot(storage, slot)
        request = RequestCache(request_id, slot, pages=[[] for _ in self.groups])
        self.requests[request_id] = request
        return request

    def get(self, request_id: Hashable) -> RequestCache:
        try:
            return self.requests[request_id]
        except KeyError:
            raise KeyError(f"request {request_id!r} is not open") from None

    def blocks_for(self, tokens: int) -> int:
        return (tokens + self.page_size - 1) // self.page_size

    def most_blocks(self, group: CacheGroup, total: int, portion: int) -> int:
        """The most pages of ``group`` that a request of ``total`` tokens holds at any time when steps bring it
        at most ``portion`` tokens."""
        whole = self.blocks_for(total)
        if group.need.window is None:
            return whole
        return min(whole, window_blocks(group.need.window, max(1, min(portion, total)), self.page_size))

    def pages_needed(self, request: RequestCache, count: int) -> List[int]:
        """Pages each group would have to take to hold ``count`` more positions."""
        total = request.num_tokens + request.reserved + count
        return [max(0, self.blocks_for(total) - len(request.pages[group.index])) for group in self.groups]

    def can_reserve(self, request: RequestCache, count: int) -> bool:
        return all(need <= group.pool.num_free
                   for need, group in zip(self.pages_needed(request, count), self.groups))

    def reserve(self, request: RequestCache, count: int) -> None:
        """Take the pages for ``count`` more positions in every group, or none at all."""
        if request.closed:
            raise KeyError(f"request {request.request_id!r} is closed")
        if count < 0:
            raise ValueError("cannot reserve a negative number of positions")
        needed = self.pages_needed(request, count)
        for need, group in zip(needed, self.groups):
            if need > group.pool.num_free:
                raise OutOfPages(f"request {request.request_id!r} needs {need} pages in group {group.index}, "
                                 f"{group.pool.num_free} free of {group.pool.num_pages}")
        for need, group in zip(needed, self.groups):
            if need:
                pages = request.pages[group.index]
                if len(pages) + need > self.max_blocks:
                    raise OutOfPages(f"request {request.request_id!r} would hold more than {self.max_blocks} blocks")
                taken = group.pool.take(need)
                group.tables[request.slot, len(pages):len(pages) + need] = taken
                pages.extend(taken)
        request.reserved += count

    def cancel_reservation(self, request: RequestCache) -> None:
        """Give back pages that only a reservation needed (a step that did not run)."""
        keep = self.blocks_for(request.num_tokens)
        for group in self.groups:
            pages = request.pages[group.index]
            extra = [page for page in pages[keep:] if page != RELEASED]
            group.pool.give(extra)
            group.tables[request.slot, keep:len(pages)] = RELEASED
            del pages[keep:]
        request.reserved = 0

    def commit(self, request: RequestCache, count: int) -> None:
        """``count`` reserved positions now hold keys and values; pages a window has passed go back."""
        if count > request.reserved:
            raise ValueError("cannot commit more positions than were reserved")
        request.num_tokens += count
        request.reserved -= count
        for group in self.groups:
            if group.need.window is None:
                continue
            first = group.first_needed_block(request.num_tokens)
            pages = request.pages[group.index]
            passed = [index for index in range(min(first, len(pages))) if pages[index] != RELEASED]
            if passed:
                group.pool.give(pages[index] for index in passed)
                for index in passed:
                    pages[index] = RELEASED
                    group.tables[request.slot, index] = RELEASED

    def close(self, request_id: Hashable) -> None:
        request = self.requests.pop(request_id, None)
        if request is None:
            raise KeyError(f"request {request_id!r} is not open")
        for group in self.groups:
            group.pool.give(page for page in request.pages[group.index] if page != RELEASED)
            group.tables[request.slot, :len(request.pages[group.index])] = RELEASED
            request.pages[group.index] = []
        self.slots.give([request.slot])
        request.closed = True

    # ---- accounting ----------------------------------------------------------------------
    def free_pages(self) -> List[int]:
        return [group.pool.num_free for group in self.groups]

    def held_pages(self) -> List[int]:
        return [group.pool.num_held for group in self.groups]

    def bytes_per_page(self, group: CacheGroup) -> int:
        return len(group.entries) * self.page_size * group.need.bytes_per_position(self.dtype)

    def state_bytes(self) -> int:
        """Bytes of the slots of every run entry that keeps per-request state, for all request slots."""
        return sum(self.max_requests * binding.need.bytes_per_request(self.dtype) for binding in self._bindings
                   if binding is not None and not binding.need.paged and binding.owned)

    def allocated_bytes(self) -> int:
        return sum(self.bytes_per_page(group) * group.pool.num_pages for group in self.groups)

    def active_bytes(self) -> int:
        return sum(self.bytes_per_page(group) * group.pool.num_held for group in self.groups)

    def check(self) -> None:
        """Every page is either free or held by exactly one request; every slot likewise."""
        for group in self.groups:
            seen: Dict[int, Hashable] = {}
            for request in self.requests.values():
                for page in request.pages[group.index]:
                    if page == RELEASED:
                        continue
                    if page in seen:
                        raise AssertionError(f"page {page} of group {group.index} is held by "
                                             f"{seen[page]!r} and {request.request_id!r}")
                    seen[page] = request.request_id
            free = group.pool.free_pages()
            if len(set(free)) != len(free):
                raise AssertionError(f"group {group.index}: a page is on the free list twice")
            if set(free) & set(seen):
                raise AssertionError(f"group {group.index}: a held page is on the free list")
            if len(free) + len(seen) != group.pool.num_pages:
                raise AssertionError(f"group {group.index}: {group.pool.num_pages - len(free) - len(seen)} pages lost")
            live_slots = {request.slot: request for request in self.requests.values()}
            for slot in range(self.max_requests):
                row = group.tables[slot]
                pages = live_slots[slot].pages[group.index] if slot in live_slots else []
                if list(row[:len(pages)]) != list(pages) or not np.all(row[len(pages):] == RELEASED):
                    raise AssertionError(f"group {group.index}: the table row of slot {slot} differs from its request's pages")
        slots = [request.slot for request in self.requests.values()]
        if len(set(slots)) != len(slots):
            raise AssertionError("two requests share a state slot")
        if len(slots) + self.slots.num_free != self.max_requests:
            raise AssertionError("a state slot is lost")
