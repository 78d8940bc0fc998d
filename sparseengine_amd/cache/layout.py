"""How keys and values lie inside a page, seen from Python.

A cache layer is ``[pages, 2 (keys, values), kv_heads, page_size, head_dim]``; the last two sizes
give a page's geometry, not the order of its elements.  Inside a kv head's page plane the elements
lie in groups of eight, so that sixteen lanes of a matrix-core operand load read one contiguous
stretch (``key_place`` / ``value_place`` in csrc/common.h):

    keys    [head_dim / 8][page_size][8]     eight dims of one key side by side, keys next to each other
    values  [page_size / 8][head_dim][8]     eight keys of one dim side by side, dims next to each other

``keys_view`` and ``values_view`` give strided views in which a key and a dim can be addressed; the
kernels never use them, tests and the kernel twins do.  ``page_size`` and ``head_dim`` are multiples
of 8.
"""
from __future__ import annotations

import torch


def keys_view(cache: torch.Tensor) -> torch.Tensor:
    """``[pages, kv_heads, page_size, head_dim / 8, 8]``: element ``[p, h, key, d // 8, d % 8]``."""
    pages, _, kv_heads, page_size, head_dim = cache.shape
    return cache[:, 0].reshape(pages, kv_heads, head_dim // 8, page_size, 8).permute(0, 1, 3, 2, 4)


def values_view(cache: torch.Tensor) -> torch.Tensor:
    """``[pages, kv_heads, page_size / 8, 8, head_dim]``: element ``[p, h, key // 8, key % 8, d]``."""
    pages, _, kv_heads, page_size, head_dim = cache.shape
    return cache[:, 1].reshape(pages, kv_heads, page_size // 8, head_dim, 8).permute(0, 1, 2, 4, 3)


def read_keys(cache: torch.Tensor, pages: torch.Tensor, offsets: torch.Tensor) -> torch.Tensor:
    """Keys at (page, offset) pairs: ``[n, kv_heads, head_dim]``."""
    return keys_view(cache)[pages, :, offsets].reshape(pages.numel(), cache.shape[2], cache.shape[4])


def read_values(cache: torch.Tensor, pages: torch.Tensor, offsets: torch.Tensor) -> torch.Tensor:
    """Values at (page, offset) pairs: ``[n, kv_heads, head_dim]``."""
    return values_view(cache)[pages, :, offsets // 8, offsets % 8]


def write_keys(cache: torch.Tensor, pages: torch.Tensor, offsets: torch.Tensor, keys: torch.Tensor) -> None:
    """``keys``: ``[n, kv_heads, head_dim]``."""
    keys_view(cache)[pages, :, offsets] = keys.reshape(pages.numel(), cache.shape[2], cache.shape[4] // 8, 8)


def write_values(cache: torch.Tensor, pages: torch.Tensor, offsets: torch.Tensor, values: torch.Tensor) -> None:
    """``values``: ``[n, kv_heads, head_dim]``."""
    values_view(cache)[pages, :, offsets // 8, offsets % 8] = values.reshape(pages.numel(), cache.shape[2], cache.shape[4])
