"""What a run entry can ask of the cache, and how each kind of need is allocated, measured and handed over.

A need is a small frozen description that a mixer returns from ``cache_need()``. The manager never looks inside
one: it asks the need itself whether it lives in pages (a block table per request, pages given back when the
request ends or a window has passed them) or in one slot of fixed size per request, lets it allocate its
storage, and hands the mixer whatever ``bind`` returns. Needs that compare equal share a group: one pool of
pages and one block table per request. A new kind of cache payload (one latent vector a token, keys alone, keys
and values of different widths) is a new subclass, defined wherever its mixer is; nothing here lists kinds.

The two kinds this package's own parts use are here: ``PagedKVNeed`` (keys and values in the tile order the MFMA
attention kernels read, see ``cache.layout``) and ``StateNeed`` (a tensor per request, zero when it opens).
The reference has one ``[slots, kv_heads, capacity, head_dim]`` tensor per layer and nothing else
(src/inference/kv_cache.cpp:11-64).
"""
from __future__ import annotations

import dataclasses
from dataclasses import dataclass
from typing import Any, List, Optional, Tuple

import torch

from .layout import check_sizes, key_page_shape, value_page_shape


def _element_size(dtype: torch.dtype) -> int:
    return torch.empty((), dtype=dtype).element_size()


class CacheNeed:
    """Base of every need. Subclasses are frozen dataclasses (hashable: equal needs share a group).

    A paged need sets ``paged = True``, may carry ``window`` (positions older than that are never read again,
    so their pages go back), and implements ``check_page_size``, ``allocate_pages`` and ``bytes_per_position``.
    A slot need leaves ``paged`` False and implements ``allocate_slots``, ``zero_slot`` and ``bytes_per_request``.
    Both implement ``bind``: what the mixer's ``forward`` receives as ``cache``; it must have ``need``, ``owned``,
    ``tensors()`` and ``shared()`` (the ``Binding`` base gives these)."""
    paged = False
    window: Optional[int] = None

    # ---- paged needs ---------------------------------------------------------------------
    def check_page_size(self, page_size: int) -> None:
        """Raise ``ValueError`` if pages of ``page_size`` positions cannot hold this need's layout."""

    def allocate_pages(self, num_pages: int, page_size: int, dtype: torch.dtype, device: torch.device) -> Any:
        raise NotImplementedError(f"{type(self).__name__} does not live in pages")

    def bytes_per_position(self, dtype: torch.dtype) -> int:
        """Bytes one position of one run entry takes in its pages."""
        raise NotImplementedError(f"{type(self).__name__} does not live in pages")

    # ---- slot needs ----------------------------------------------------------------------
    def allocate_slots(self, max_requests: int, dtype: torch.dtype, device: torch.device) -> Any:
        raise NotImplementedError(f"{type(self).__name__} does not live in request slots")

    def zero_slot(self, storage: Any, slot: int) -> None:
        """A request opens in ``slot``: make the slot what a fresh request must find."""
        raise NotImplementedError(f"{type(self).__name__} does not live in request slots")

    def bytes_per_request(self, dtype: torch.dtype) -> int:
        raise NotImplementedError(f"{type(self).__name__} does not live in request slots")

    # ---- both ----------------------------------------------------------------------------
    def bind(self, group: Optional[int], storage: Any, owned: bool) -> "Binding":
        """What the mixer gets: ``group`` indexes ``ctx.paged`` (None for a slot need), ``storage`` is what the
        allocation returned (None where the manager only keeps books, without a device)."""
        raise NotImplementedError


@dataclass
class Binding:
    """What a mixer's forward receives as ``cache``. ``owned`` is False for a run entry that reads another's."""
    need: CacheNeed
    owned: bool = True

    def tensors(self) -> List[torch.Tensor]:
        """The device tensors behind this binding (for accounting, and for filling a cache with stand-in data)."""
        return []

    def shared(self) -> "Binding":
        """The same storage for a run entry that reads it without owning it."""
        return dataclasses.replace(self, owned=False)


# ---- keys and values in pages ------------------------------------------------------------------
@dataclass(frozen=True)
class PagedKVNeed(CacheNeed):
    """Keys and values in pages; ``window`` is None when every key stays needed."""
    kv_heads: int
    head_dim: int
    window: Optional[int] = None
    paged = True

    def check_page_size(self, page_size: int) -> None:
        check_sizes(page_size, self.head_dim)     # pages are tiled by 16 positions

    def allocate_pages(self, num_pages, page_size, dtype, device):
        # Zeroed once: a kernel may read a whole tile whose tail was never written.
        k = torch.zeros(key_page_shape(num_pages, self.kv_heads, page_size, self.head_dim), dtype=dtype, device=device)
        v = torch.zeros(value_page_shape(num_pages, self.kv_heads, page_size, self.head_dim), dtype=dtype, device=device)
        return k, v

    def bytes_per_position(self, dtype):
        return 2 * self.kv_heads * self.head_dim * _element_size(dtype)

    def bind(self, group, storage, owned):
        k, v = storage if storage is not None else (None, None)
        return PagedBinding(self, owned, group, k, v)


@dataclass
class PagedBinding(Binding):
    """What a mixer gets for paged keys and values: its entry's page arrays and its group."""
    group: int = 0
    k: Optional[torch.Tensor] = None
    v: Optional[torch.Tensor] = None

    def tensors(self):
        return [tensor for tensor in (self.k, self.v) if tensor is not None]


# ---- per-request state of fixed size -------------------------------------------------------------
@dataclass(frozen=True)
class StateNeed(CacheNeed):
    """Per-request state of fixed size: one slot of ``shape`` and ``dtype`` per live request."""
    shape: Tuple[int, ...]
    dtype: torch.dtype = torch.float32

    def allocate_slots(self, max_requests, dtype, device):
        return torch.zeros((max_requests, *self.shape), dtype=self.dtype, device=device)

    def zero_slot(self, storage, slot):
        storage[slot].zero_()

    def bytes_per_request(self, dtype):
        count = 1
        for size in self.shape:
            count *= int(size)
        return count * _element_size(self.dtype)

    def bind(self, group, storage, owned):
        return StateBinding(self, owned, storage)


@dataclass
class StateBinding(Binding):
    """What a mixer gets for per-request state: ``state[slot]`` is the request's, zero when it opens."""
    state: Optional[torch.Tensor] = None

    def tensors(self):
        return [self.state] if self.state is not None else []
