"""The shapes of key and value pages, and views that show them as plain ``[page, kv_head, position, dim]``.

Pages hold their positions in tiles of 16, laid out in the order the MFMA kernels read them (the same
formulas are in ``csrc/cache_layout.h``):

    keys:   [page, kv_head, tile, dim // 8, position % 16, dim % 8]
    values: [page, kv_head, tile, dim // 32, (position % 16) // 8, dim % 32, position % 8], the tile flat
            (a last block of 16 dims, where ``head_dim`` is an odd multiple of 16, is [position // 8, 16, 8])

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
    return (num_pages, kv_heads, page_size // TILE, -(-head_dim // 16) * 16 * TILE)


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


def value_index(dims: int) -> torch.Tensor:
    """Where (position, dim) of a tile lies in the flat tile, ``[TILE, dims]``; ``dims`` is a multiple of 16."""
    position = torch.arange(TILE).view(TILE, 1)
    dim = torch.arange(dims).view(1, dims)
    block = dim // 32
    width = torch.clamp(dims - 32 * block, max=32)
    return block * 512 + ((position // 8) * width + dim % 32) * 8 + position % 8


class _ValueView:
    def __init__(self, pages: torch.Tensor, head_dim: int):
        self.pages, self.head_dim = pages, head_dim
        self.dims = pages.shape[-1] // TILE
        self.index = value_index(self.dims).to(pages.device)

    def read(self) -> torch.Tensor:
        pages, kv_heads, tiles, _ = self.pages.shape
        plain = self.pages[..., self.index]      # [page, kv_head, tile, position16, dim]
        return plain.reshape(pages, kv_heads, tiles * TILE, self.dims)[..., :self.head_dim]

    def write(self, rows: torch.Tensor) -> None:
        pages, kv_heads, tiles, _ = self.pages.shape
        padded = torch.zeros((pages, kv_heads, tiles * TILE, self.dims), dtype=self.pages.dtype, device=self.pages.device)
        padded[..., :self.head_dim] = rows
        self.pages[..., self.index] = padded.view(pages, kv_heads, tiles, TILE, self.dims)


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
