"""The pages themselves: device tensors per cache group and per cache-owning step of the schedule.

Layout (chosen for the MFMA attention kernels of gfx950, not the reference's
[pages, block_size, kv_heads, d] of pagedllm/kv_cache.py:1-7):

    K pages  [pages, kv_heads, block_size, d]    one head's keys of a page are contiguous rows
    V pages  [pages, kv_heads, d, block_size]    transposed inside the page, so that 8 successive
                                                 positions of one channel are one 16-byte load, the
                                                 operand shape of the P*V matrix instruction

A slot is ``page * block_size + offset`` as in the reference.
"""

from __future__ import annotations

from dataclasses import dataclass

import torch

from ..csrc import ops
from ..parts.base import CacheSpec
from .block_manager import PageCopy


@dataclass
class LayerCache:
    k_pages: torch.Tensor
    v_pages: torch.Tensor
    group: str
    block_size: int
    num_pages: int
    writable: bool = True

    def read_only(self) -> "LayerCache":
        return LayerCache(self.k_pages, self.v_pages, self.group, self.block_size, self.num_pages, writable=False)


@dataclass
class CacheGroup:
    name: str
    spec: CacheSpec
    owners: list          # schedule steps that own pages in this group

    def bytes_per_page(self, block_size: int, dtype: torch.dtype) -> int:
        elem = torch.empty((), dtype=dtype).element_size()
        return 2 * len(self.owners) * block_size * self.spec.num_kv_heads * self.spec.head_dim * elem


class KVCacheStorage:
    def __init__(self, groups: dict, num_pages: int | dict, block_size: int, dtype: torch.dtype, device):
        self.groups = groups
        self.block_size = block_size
        self.dtype = dtype
        self.device = torch.device(device)
        self.num_pages = {g: (num_pages[g] if isinstance(num_pages, dict) else num_pages) for g in groups}
        self._layers: dict[int, LayerCache] = {}
        for name, group in groups.items():
            n, s = self.num_pages[name], group.spec
            for owner in group.owners:
                k = torch.zeros((n, s.num_kv_heads, block_size, s.head_dim), dtype=dtype, device=self.device)
                v = torch.zeros((n, s.num_kv_heads, s.head_dim, block_size), dtype=dtype, device=self.device)
                self._layers[owner] = LayerCache(k, v, name, block_size, n)

    def for_step(self, owner: int, writable: bool = True) -> LayerCache:
        c = self._layers[owner]
        return c if writable else c.read_only()

    def apply_copies(self, copies: dict) -> None:
        """Copy-on-write page copies, for every owner of the group (pagedllm/kv_cache.py:47-54)."""
        for name, ops_list in copies.items():
            if not ops_list:
                continue
            src = torch.tensor([c.src for c in ops_list], dtype=torch.int32, device=self.device)
            dst = torch.tensor([c.dst for c in ops_list], dtype=torch.int32, device=self.device)
            for owner in self.groups[name].owners:
                c = self._layers[owner]
                ops.copy_pages(c.k_pages, src, dst)
                ops.copy_pages(c.v_pages, src, dst)

    def total_bytes(self) -> int:
        return sum(c.k_pages.numel() * c.k_pages.element_size() * 2 for c in self._layers.values())
