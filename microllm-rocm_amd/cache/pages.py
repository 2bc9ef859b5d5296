"""Pools of pages and of state slots: plain bookkeeping, no device memory.

A page is an index into a group's page arrays; a pool hands pages out and takes
them back, refuses a page that is given back twice or was never taken, and can
list what is free and what is held, so tests can check that no page is lost or
held twice. Pages that were given back last are handed out first, so reuse
happens as early as it can.
"""
from __future__ import annotations

from typing import Iterable, List


class OutOfPages(RuntimeError):
    """A pool cannot give what was asked for; nothing was taken."""


class PagePool:
    def __init__(self, num_pages: int):
        if num_pages <= 0:
            raise ValueError("a pool needs at least one page")
        self.num_pages = num_pages
        self._free: List[int] = list(range(num_pages - 1, -1, -1))  # a stack; page 0 goes out first
        self._held = bytearray(num_pages)
        self.peak_held = 0
        self.total_taken = 0

    @property
    def num_free(self) -> int:
        return len(self._free)

    @property
    def num_held(self) -> int:
        return self.num_pages - len(self._free)

    def take(self, count: int) -> List[int]:
        if count < 0:
            raise ValueError("cannot take a negative number of pages")
        if count > len(self._free):
            raise OutOfPages(f"{count} pages wanted, {len(self._free)} free of {self.num_pages}")
        pages = [self._free.pop() for _ in range(count)]
        for page in pages:
            self._held[page] = 1
        self.total_taken += count
        self.peak_held = max(self.peak_held, self.num_held)
        return pages

    def give(self, pages: Iterable[int]) -> None:
        pages = list(pages)
        for page in pages:
            if not 0 <= page < self.num_pages:
                raise ValueError(f"page {page} does not belong to this pool")
            if not self._held[page]:
                raise ValueError(f"page {page} is given back but is not held")
            self._held[page] = 0
            self._free.append(page)

    def free_pages(self) -> List[int]:
        return list(self._free)

    def held_pages(self) -> List[int]:
        return [page for page in range(self.num_pages) if self._held[page]]


class SlotPool(PagePool):
    """Slots for per-request state of fixed size: one per live request."""

    def take_one(self) -> int:
        try:
            return self.take(1)[0]
        except OutOfPages:
            raise OutOfPages(f"all {self.num_pages} request slots are in use") from None
