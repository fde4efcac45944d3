"""Device storage behind the cache manager: for every cache-owning call the page tensors its
mixer declares (``CacheSpec.pages``), each ``[num_blocks, *page shape]``, and state tensors
``[num_slots, *shape]`` for mixers with fixed-size state.  Attention declares K pages
``[kv_heads, block_size, head_dim]`` (one (page, head) tile is contiguous, a key's elements side
by side) and V pages transposed, ``[kv_heads, head_dim, block_size]`` (an element's keys side by
side), which is the order the matrix cores contract ``P * V`` in.  The reference keeps
``[num_blocks, block_size, kv_heads, head_dim]`` for both (src/tokenvault/cache/kv_cache.py:27-31).
"""

from __future__ import annotations

import torch

from kvforge_amd.cache.manager import CacheGroup
from kvforge_amd.parts.base import StateSpec


class PagedStorage:
    def __init__(self, groups: list[CacheGroup], num_blocks: list[int], block_size: int,
                 dtype: torch.dtype, device: torch.device | str) -> None:
        self.block_size, self.dtype = block_size, dtype
        self.pages: dict[int, dict[str, torch.Tensor]] = {}    # owning call -> name -> tensor
        self.group_of: dict[int, int] = {}
        for g, (grp, nb) in enumerate(zip(groups, num_blocks)):
            for layer in grp.layers:
                self.pages[layer] = {
                    t.name: torch.zeros((nb, *t.page_shape(block_size)), dtype=t.dtype or dtype,
                                        device=device) for t in grp.pages}
                self.group_of[layer] = g

    @property
    def memory_bytes(self) -> int:
        return sum(t.numel() * t.element_size() for held in self.pages.values() for t in held.values())


class StateStorage:
    def __init__(self, specs: dict[int, StateSpec], num_slots: int,
                 device: torch.device | str) -> None:
        self.tensors = {layer: torch.zeros((num_slots, *s.shape), dtype=s.dtype, device=device)
                        for layer, s in specs.items()}


def bytes_per_block(groups: list[CacheGroup], block_size: int, dtype: torch.dtype) -> int:
    """What one page number costs over every layer of every group: for attention K and V,
    ``2 * layers * block_size * kv_heads * head_dim * element size``
    (src/tokenvault/config.py:91-95)."""
    return sum(len(g.layers) * sum(t.page_bytes(block_size, dtype) for t in g.pages) for g in groups)
