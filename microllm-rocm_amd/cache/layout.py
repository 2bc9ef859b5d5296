"""The shapes of key and value pages, and views that show them as plain ``[page, kv_head, position, dim]``.

Pages hold their positions in tiles of 16, laid out in the order the MFMA kernels read them (the same
formulas are in ``csrc/cache_layout.h``):

    keys:   [page, kv_head, tile, dim // 8, position % 16, dim % 8]
    values: [page, kv_head, tile, dim // 16, (position % 16) // 4, dim % 16, position % 4]

``head_dim`` is padded to a multiple of 8 (keys) or 16 (values).
"""
from __future__ import annotations

from typing import Tuple

import torch

TILE = 16


def check_sizes(page_size: int, head_dim: int) -> None:
    if page_size <= 0 or page_size % TILE != 0:
        raise ValueError(f"page_size must be a positive multiple of {TILE}, got {page_size}")
    if head_dim <= 0:
        raise ValueError("head_dim must be positive")


def key_page_shape(num_pages: int, kv_heads: int, page_size: int, head_dim: int) -> Tuple[int, ...]:
    check_sizes(page_size, head_dim)
    return (num_pages, kv_heads, page_size // TILE, -(-head_dim // 8), TILE, 8)


def value_page_shape(num_pages: int, kv_heads: int, page_size: int, head_dim: int) -> Tuple[int, ...]:
    check_sizes(page_size, head_dim)
    return (num_pages, kv_heads, page_size // TILE, -(-head_dim // 16), 4, TILE, 4)


class _KeyView:
    """Indexable as ``view[page, :, offset, :]`` for reading and writing single positions."""

    def __init__(self, pages: torch.Tensor, head_dim: int):
        self.pages, self.head_dim = pages, head_dim

    def _plain(self) -> torch.Tensor:
        pages, kv_heads, tiles, chunks, _, _ = self.pages.shape
        return self.pages.permute(0, 1, 2, 4, 3, 5)   # [page, kv_head, tile, position16, chunk, 8]

    def read(self) -> torch.Tensor:
        pages, kv_heads, tiles, chunks, _, _ = self.pages.shape
        return self._plain().reshape(pages, kv_heads, tiles * TILE, chunks * 8)[..., :self.head_dim]

    def write(self, rows: torch.Tensor) -> None:
        """``rows``: ``[page, kv_head, position, head_dim]`` written into the pages."""
        pages, kv_heads, tiles, chunks, _, _ = self.pages.shape
        padded = torch.zeros((pages, kv_heads, tiles * TILE, chunks * 8), dtype=self.pages.dtype, device=self.pages.device)
        padded[..., :self.head_dim] = rows
        self._plain().copy_(padded.view(pages, kv_heads, tiles, TILE, chunks, 8))


class _ValueView:
    def __init__(self, pages: torch.Tensor, head_dim: int):
        self.pages, self.head_dim = pages, head_dim

    def _plain(self) -> torch.Tensor:
        # [page, kv_head, tile, dim_tile, quad, dim16, key4] -> [page, kv_head, tile, quad, key4, dim_tile, dim16]
        return self.pages.permute(0, 1, 2, 4, 6, 3, 5)

    def read(self) -> torch.Tensor:
        pages, kv_heads, tiles, dim_tiles, _, _, _ = self.pages.shape
        return self._plain().reshape(pages, kv_heads, tiles * TILE, dim_tiles * 16)[..., :self.head_dim]

    def write(self, rows: torch.Tensor) -> None:
        pages, kv_heads, tiles, dim_tiles, _, _, _ = self.pages.shape
        padded = torch.zeros((pages, kv_heads, tiles * TILE, dim_tiles * 16), dtype=self.pages.dtype, device=self.pages.device)
        padded[..., :self.head_dim] = rows
        self._plain().copy_(padded.view(pages, kv_heads, tiles, 4, 4, dim_tiles, 16))


def key_rows(k_pages: torch.Tensor, head_dim: int) -> torch.Tensor:
    """Keys as ``[page, kv_head, position, dim]`` (a copy)."""
    return _KeyView(k_pages, head_dim).read()


def value_rows(v_pages: torch.Tensor, head_dim: int) -> torch.Tensor:
    """Values as ``[page, kv_head, position, dim]`` (a copy)."""
    return _ValueView(v_pages, head_dim).read()


def write_key_rows(k_pages: torch.Tensor, rows: torch.Tensor) -> None:
    _KeyView(k_pages, rows.shape[-1]).write(rows)


def write_value_rows(v_pages: torch.Tensor, rows: torch.Tensor) -> None:
    _ValueView(v_pages, rows.shape[-1]).write(rows)
