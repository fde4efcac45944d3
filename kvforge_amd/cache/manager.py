"""Cache manager: pages and per-request block tables for every cache group, and slots for
per-request state of fixed size.  Pure Python, no tensors.

Compared with the reference's ``BlockManager`` (src/tokenvault/cache/block_manager.py:55-314):
the same allocate / can_allocate / can_append_slots / append_slots / free life cycle, slot
addressing ``table[pos // bs] * bs + pos % bs`` and watermark; no prefix-cache hashing.  New
here: several *groups* of layers (one that keeps every key, one that keeps a window of them, ...)
each with a pool and tables of its own, early return of pages a window has passed, and
``StateSlots``.
"""

from __future__ import annotations

from dataclasses import dataclass

from kvforge_amd.cache.block_pool import BlockPool, NoFreeBlocksError

RELEASED = -1  # table entry of a page that was given back (or never held)


@dataclass(frozen=True)
class CacheGroup:
    """Layers whose mixers have equal cache needs.  ``layers``: places in the model's run order
    of the calls that own pages in this group; ``pages``: the tensors a page consists of, as
    the mixers declare them (``parts.base.PageTensor``; the manager itself only counts pages
    and never looks at them)."""

    layers: tuple[int, ...]
    pages: tuple = ()
    window: int | None = None


@dataclass(frozen=True)
class CacheStats:
    num_blocks: int
    num_used_blocks: int
    num_free_blocks: int
    num_tokens: int
    utilization: float
    internal_fragmentation: float


class StateSlots:
    """Fixed-size per-request state: a slot is taken when a request is admitted and returned when
    it finishes or is preempted (its state is then rebuilt with its tokens)."""

    def __init__(self, num_slots: int) -> None:
        self.num_slots = int(num_slots)
        self._free = list(range(self.num_slots - 1, -1, -1))
        self._owner: dict[str, int] = {}

    @property
    def num_free(self) -> int:
        return len(self._free)

    def has(self, request_id: str) -> bool:
        return request_id in self._owner

    def slot(self, request_id: str) -> int:
        return self._owner[request_id]

    def take(self, request_id: str) -> int:
        if request_id in self._owner:
            raise ValueError(f"request {request_id} already holds a state slot")
        if not self._free:
            raise NoFreeBlocksError("no free state slot")
        s = self._free.pop()
        self._owner[request_id] = s
        return s

    def release(self, request_id: str) -> None:
        s = self._owner.pop(request_id, None)
        if s is not None:
            self._free.append(s)


class CacheManager:
    def __init__(self, block_size: int, groups: list[CacheGroup], num_blocks: "int | list[int]",
                 num_state_slots: int = 0, watermark: float = 0.0) -> None:
        if block_size <= 0:
            raise ValueError("block_size must be positive")
        self.block_size = int(block_size)
        self.groups = list(groups)
        counts = [num_blocks] * len(self.groups) if isinstance(num_blocks, int) else list(num_blocks)
        if len(counts) != len(self.groups):
            raise ValueError("one page count per cache group is needed")
        self.pools = [BlockPool(n) for n in counts]
        self.watermark_blocks = [int(watermark * n) for n in counts]
        self._tables: list[dict[str, list[int]]] = [{} for _ in self.groups]
        # per group and request: pages [0, n) of the table have been given back (windows only)
        self._released: list[dict[str, int]] = [{} for _ in self.groups]
        self._num_tokens: dict[str, int] = {}
        # a number per allocation, so that a request id used again is told from its former self
        self._serial: dict[str, int] = {}
        self._next_serial = 0
        self.slots = StateSlots(num_state_slots)

    # ------------------------------------------------------------------ queries
    @property
    def num_groups(self) -> int:
        return len(self.groups)

    @property
    def num_blocks(self) -> int:
        """Pages of the smallest pool: what bounds a request that needs every position."""
        return min((p.num_blocks for p in self.pools), default=0)

    @property
    def num_free_blocks(self) -> int:
        return min((p.num_free for p in self.pools), default=0)

    def has_request(self, request_id: str) -> bool:
        return request_id in self._num_tokens

    def num_tokens(self, request_id: str) -> int:
        return self._num_tokens[request_id]

    def serial(self, request_id: str) -> int:
        """Changes whenever ``request_id`` is allocated anew."""
        return self._serial[request_id]

    def block_table(self, request_id: str, group: int = 0) -> list[int]:
        return self._tables[group][request_id]

    def blocks_needed(self, num_tokens: int) -> int:
        return -(-num_tokens // self.block_size)

    def slot(self, request_id: str, position: int, group: int = 0) -> int:
        """Flat slot ``page * block_size + offset`` of a position
        (src/tokenvault/cache/block_manager.py:101-104)."""
        t = self._tables[group][request_id]
        return t[position // self.block_size] * self.block_size + position % self.block_size

    def _first_live_block(self, g: int, first_query_pos: int) -> int:
        w = self.groups[g].window
        if w is None:
            return 0
        return max(0, first_query_pos - w + 1) // self.block_size

    def _new_blocks(self, g: int, request_id: str | None, total_tokens: int) -> int:
        """Pages group ``g`` must take to back positions up to ``total_tokens``.  A table only
        grows at its end (pages a window has passed are never taken back), so this is the number
        of entries it lacks."""
        need = self.blocks_needed(total_tokens)
        have = len(self._tables[g][request_id]) if request_id is not None else 0
        return max(0, need - have)

    # --------------------------------------------------------------- life cycle
    def can_allocate(self, num_tokens: int, reserve: bool = True) -> bool:
        """Room for a new request of ``num_tokens`` while keeping the watermark free
        (src/tokenvault/cache/block_manager.py:165-170); ``reserve=False`` leaves the watermark
        out, for a pool that is as empty as it will ever get."""
        if self.slots.num_slots and self.slots.num_free == 0:
            return False
        return all(self._new_blocks(g, None, num_tokens) <= p.num_free - (wm if reserve else 0)
                   for g, (p, wm) in enumerate(zip(self.pools, self.watermark_blocks)))

    def allocate(self, request_id: str, num_tokens: int) -> None:
        """Tables for a new request covering ``num_tokens`` positions, and a state slot."""
        if request_id in self._num_tokens:
            raise ValueError(f"request {request_id} already allocated")
        for g, p in enumerate(self.pools):
            if self._new_blocks(g, None, num_tokens) > p.num_free:
                raise NoFreeBlocksError(f"cannot allocate {num_tokens} tokens for {request_id}")
        if self.slots.num_slots:
            self.slots.take(request_id)
        for g in range(len(self.groups)):
            self._tables[g][request_id] = []
            self._released[g][request_id] = 0
        self._num_tokens[request_id] = 0
        self._serial[request_id] = self._next_serial
        self._next_serial += 1
        self.append_slots(request_id, num_tokens, 0)

    def can_append_slots(self, request_id: str, total_tokens: int, write_start: int) -> bool:
        """Room to grow ``request_id`` to ``total_tokens`` positions, no watermark
        (src/tokenvault/cache/block_manager.py:204-207)."""
        for g, p in enumerate(self.pools):
            if self._new_blocks(g, request_id, total_tokens) > p.num_free:
                return False
        return True

    def can_append_all(self, wanted: "list[tuple[str, int]]") -> bool:
        """Room to grow every ``(request_id, total_tokens)`` of ``wanted`` at once."""
        for g, p in enumerate(self.pools):
            if sum(self._new_blocks(g, rid, total) for rid, total in wanted) > p.num_free:
                return False
        return True

    def append_slots(self, request_id: str, total_tokens: int, write_start: int) -> None:
        """Back every position in ``[write_start, total_tokens)`` (and what those queries still
        see) with pages.  All-or-nothing: raises before taking anything if a pool is short."""
        need = self.blocks_needed(total_tokens)
        short = [g for g in range(len(self.pools)) if len(self._tables[g][request_id]) < need]
        if short:
            if not self.can_append_slots(request_id, total_tokens, write_start):
                raise NoFreeBlocksError(f"cannot append slots for {request_id}")
            for g in short:
                p, table = self.pools[g], self._tables[g][request_id]
                while len(table) < need:
                    table.append(p.take())
        if total_tokens > self._num_tokens[request_id]:
            self._num_tokens[request_id] = total_tokens

    def release_behind(self, request_id: str, num_computed: int) -> int:
        """Give back pages of windowed groups that no later query can see: the next query sits at
        position ``num_computed`` and sees keys from ``num_computed - window + 1`` on.  Returns
        how many pages were given back."""
        n = 0
        for g, p in enumerate(self.pools):
            if self.groups[g].window is None:
                continue
            table = self._tables[g].get(request_id)
            if table is None:
                continue
            upto = min(self._first_live_block(g, num_computed), len(table))
            for i in range(self._released[g][request_id], upto):
                if table[i] != RELEASED:
                    p.release(table[i])
                    table[i] = RELEASED
                    n += 1
            if upto > self._released[g][request_id]:
                self._released[g][request_id] = upto
        return n

    def free(self, request_id: str) -> None:
        """Give back everything the request holds; unknown requests are a no-op
        (src/tokenvault/cache/block_manager.py:268-276)."""
        if self._num_tokens.pop(request_id, None) is None:
            return
        self._serial.pop(request_id, None)
        for g, p in enumerate(self.pools):
            self._released[g].pop(request_id, None)
            for b in reversed(self._tables[g].pop(request_id)):
                if b != RELEASED:
                    p.release(b)
        self.slots.release(request_id)

    def mark_computed(self, request_id: str, num_tokens: int) -> None:
        """Record the live token count (stats only; src/tokenvault/cache/block_manager.py:249-253)."""
        if request_id in self._num_tokens:
            self._num_tokens[request_id] = num_tokens

    # ------------------------------------------------------------------ metrics
    def stats(self, group: int = 0) -> CacheStats:
        p = self.pools[group]
        used = p.num_used
        tokens = 0
        bs = self.block_size
        for rid, table in self._tables[group].items():
            n = self._num_tokens[rid]
            for i, b in enumerate(table):
                if b != RELEASED:
                    tokens += min(bs, max(0, n - i * bs))
        slots = used * bs
        return CacheStats(p.num_blocks, used, p.num_free, tokens, used / p.num_blocks,
                          (1.0 - tokens / slots) if slots else 0.0)
