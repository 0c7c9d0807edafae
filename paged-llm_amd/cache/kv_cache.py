"""The pages themselves: device tensors per cache group and per cache-owning step of the schedule.

What a page holds is the mixer's to say (``parts.base.CacheSpec.tensors``): for every tensor it names, each owner
gets one device tensor ``[pages, *page shape]``, where the page shape has the page's positions wherever the mixer
put them.  (The reference has one fixed pair, K and V as [pages, block_size, kv_heads, d], pagedllm/kv_cache.py:34-40;
the attention part here declares K ``[kv_heads, block_size, d]`` and V ``[kv_heads, d, block_size]``, the layouts its
matrix-core kernels load straight into operand registers.)

A slot is ``page * block_size + offset`` as in the reference.
"""

from __future__ import annotations

from dataclasses import dataclass

import torch

from ..csrc import ops
from ..parts.base import CacheSpec


@dataclass
class LayerCache:
    """The page tensors of one cache-owning step, by the names its mixer gave them."""
    tensors: dict             # name -> [pages, *page shape]
    group: str
    block_size: int
    num_pages: int
    writable: bool = True

    def __getitem__(self, name: str) -> torch.Tensor:
        return self.tensors[name]

    def read_only(self) -> "LayerCache":
        return LayerCache(self.tensors, self.group, self.block_size, self.num_pages, writable=False)


@dataclass
class CacheGroup:
    name: str
    spec: CacheSpec
    owners: list          # schedule steps that own pages in this group

    def bytes_per_page(self, block_size: int, dtype: torch.dtype) -> int:
        """Device bytes that one page id of this group stands for: every owner's tensors of that page."""
        return len(self.owners) * self.spec.bytes_per_page(block_size, dtype)


class KVCacheStorage:
    def __init__(self, groups: dict, num_pages: int | dict, block_size: int, dtype: torch.dtype, device):
        self.groups = groups
        self.block_size = block_size
        self.dtype = dtype
        self.device = torch.device(device)
        self.num_pages = {g: (num_pages[g] if isinstance(num_pages, dict) else num_pages) for g in groups}
        self._layers: dict[int, LayerCache] = {}
        for name, group in groups.items():
            n = self.num_pages[name]
            for owner in group.owners:
                tensors = {t.name: torch.zeros((n, *t.page_shape(block_size)), dtype=t.dtype or dtype, device=self.device)
                           for t in group.spec.tensors}
                self._layers[owner] = LayerCache(tensors, name, block_size, n)

    def for_step(self, owner: int, writable: bool = True) -> LayerCache:
        c = self._layers[owner]
        return c if writable else c.read_only()

    def apply_copies(self, copies: dict) -> None:
        """Copy-on-write page copies, for every tensor of every owner of the group (pagedllm/kv_cache.py:47-54)."""
        for name, ops_list in copies.items():
            if not ops_list:
                continue
            src = torch.tensor([c.src for c in ops_list], dtype=torch.int32, device=self.device)
            dst = torch.tensor([c.dst for c in ops_list], dtype=torch.int32, device=self.device)
            for owner in self.groups[name].owners:
                for pages in self._layers[owner].tensors.values():
                    ops.copy_pages(pages, src, dst)

    def total_bytes(self) -> int:
        return sum(t.numel() * t.element_size() for c in self._layers.values() for t in c.tensors.values())
