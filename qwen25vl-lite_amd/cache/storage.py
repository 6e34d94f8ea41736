"""The device tensors behind the cache manager's pages and slots."""

from __future__ import annotations

from typing import List, Sequence

import torch

from .manager import CacheGroupSpec

__all__ = ["KVStorage"]


class KVStorage:
    """Keys and values of every group: per group ``k`` of ``[layers, pages, nkv, page_size, hd]``
    and ``v`` of ``[layers, pages, nkv, hd, page_size]``.  One kv head's keys of a page are a
    contiguous ``page_size x hd`` tile; values are kept transposed so that the matrix-core
    kernels read eight consecutive keys of one channel with a single 16-byte load.
    The logical content is the reference's ``[layers, blocks, block_size, kv_heads, head_dim]``
    (reference src/qwen25vl_lite/cache.py:423-431)."""

    def __init__(self, groups: Sequence[CacheGroupSpec], num_pages: int, page_size: int, dtype: torch.dtype,
                 device: torch.device):
        self.page_size = page_size
        self.num_pages = num_pages
        self.k: List[torch.Tensor] = []
        self.v: List[torch.Tensor] = []
        for g in groups:
            nkv, hd = g.need.num_kv_heads, g.need.head_dim
            self.k.append(torch.zeros((g.num_layers, num_pages, nkv, page_size, hd), dtype=dtype, device=device))
            self.v.append(torch.zeros((g.num_layers, num_pages, nkv, hd, page_size), dtype=dtype, device=device))

    def copy_pages(self, group: int, src: Sequence[int], dst: Sequence[int]) -> None:
        """Keys and values of pages ``src`` into pages ``dst`` of a group, in all of its layers
        (reference cache.py:537-545)."""
        from ..ops import kernels
        kernels.copy_pages(self.k[group], src, dst)
        kernels.copy_pages(self.v[group], src, dst)

    def nbytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in self.k + self.v)
