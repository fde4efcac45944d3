"""Device storage behind the cache manager: K and V pages per cache-owning call, and state
tensors ``[num_slots, *shape]`` for mixers with fixed-size state.  K pages are
``[num_blocks, kv_heads, block_size, head_dim]`` (one (page, head) tile is contiguous, a key's
elements side by side); V pages are transposed, ``[num_blocks, kv_heads, head_dim, block_size]``
(an element's keys side by side), which is the order the matrix cores contract ``P * V`` in.
The reference keeps ``[num_blocks, block_size, kv_heads, head_dim]`` for both
(src/tokenvault/cache/kv_cache.py:27-31).
"""

from __future__ import annotations

import torch

from kvforge_amd.cache.manager import CacheGroup
from kvforge_amd.parts.base import StateSpec


class PagedStorage:
    def __init__(self, groups: list[CacheGroup], num_blocks: list[int], block_size: int,
                 dtype: torch.dtype, device: torch.device | str) -> None:
        self.block_size, self.dtype = block_size, dtype
        self.k: dict[int, torch.Tensor] = {}
        self.v: dict[int, torch.Tensor] = {}
        self.group_of: dict[int, int] = {}
        for g, (grp, nb) in enumerate(zip(groups, num_blocks)):
            k_shape = (nb, grp.num_kv_heads, block_size, grp.head_dim)
            v_shape = (nb, grp.num_kv_heads, grp.head_dim, block_size)
            for layer in grp.layers:
                self.k[layer] = torch.zeros(k_shape, dtype=dtype, device=device)
                self.v[layer] = torch.zeros(v_shape, dtype=dtype, device=device)
                self.group_of[layer] = g

    @property
    def memory_bytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in list(self.k.values()) + list(self.v.values()))


class StateStorage:
    def __init__(self, specs: dict[int, StateSpec], num_slots: int,
                 device: torch.device | str) -> None:
        self.tensors = {layer: torch.zeros((num_slots, *s.shape), dtype=s.dtype, device=device)
                        for layer, s in specs.items()}


def bytes_per_block(groups: list[CacheGroup], block_size: int, dtype: torch.dtype) -> int:
    """K and V of one page over every layer of every group (src/tokenvault/config.py:91-95)."""
    elem = torch.tensor([], dtype=dtype).element_size()
    return sum(2 * len(g.layers) * block_size * g.num_kv_heads * g.head_dim * elem for g in groups)
