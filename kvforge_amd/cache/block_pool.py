"""A pool of physical pages with reference counts (src/tokenvault/cache/block_manager.py:72-74,
114-138 without the prefix-cache hashing): a LIFO free list that hands out page 0 first, a count
per page, and a guard against freeing a page twice."""

from __future__ import annotations


class NoFreeBlocksError(RuntimeError):
    pass


class BlockPool:
    def __init__(self, num_blocks: int) -> None:
        if num_blocks <= 0:
            raise ValueError("num_blocks must be positive")
        self.num_blocks = int(num_blocks)
        self._ref = [0] * self.num_blocks
        self._free = list(range(self.num_blocks - 1, -1, -1))

    @property
    def num_free(self) -> int:
        return len(self._free)

    @property
    def num_used(self) -> int:
        return self.num_blocks - len(self._free)

    def ref_count(self, block: int) -> int:
        return self._ref[block]

    def take(self) -> int:
        if not self._free:
            raise NoFreeBlocksError("cache pool exhausted")
        b = self._free.pop()
        self._ref[b] = 1
        return b

    def share(self, block: int) -> None:
        if self._ref[block] <= 0:
            raise RuntimeError(f"page {block} is not held")
        self._ref[block] += 1

    def release(self, block: int) -> None:
        if not 0 <= block < self.num_blocks or self._ref[block] <= 0:
            raise RuntimeError(f"double free of page {block}")
        self._ref[block] -= 1
        if self._ref[block] == 0:
            self._free.append(block)
