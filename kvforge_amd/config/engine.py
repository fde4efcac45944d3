"""Engine-side configuration: cache geometry, scheduler budgets, device and dtype.

Names, defaults and post-init rules follow the reference (src/tokenvault/config.py:75-151):
``block_size=16``, ``num_blocks=256`` or derived from ``kv_cache_memory_gb``, ``watermark=0.01``;
``max_num_seqs=32``, ``max_num_batched_tokens=2048``, ``max_model_len=2048``, FCFS, chunked
prefill on; ``max_model_len`` is clamped to the model's ``max_position_embeddings``.
The device default is the GPU: this engine has no CPU path.
"""

from __future__ import annotations

import math
from dataclasses import dataclass, field
from enum import Enum

import torch

DTYPES: dict[str, torch.dtype] = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def parse_dtype(name: "str | torch.dtype") -> torch.dtype:
    if isinstance(name, torch.dtype):
        if name not in DTYPES.values():
            raise ValueError(f"engine dtype must be one of {sorted(DTYPES)}, got {name}")
        return name
    try:
        return DTYPES[name]
    except KeyError:
        raise ValueError(f"engine dtype must be one of {sorted(DTYPES)}, got {name!r}") from None


class SchedulingPolicy(str, Enum):
    """The order of the line (src/tokenvault/config.py:16-18): by arrival, or by the request's
    ``priority`` first (a smaller number is served sooner) and by arrival within one priority."""
    FCFS = "fcfs"
    PRIORITY = "priority"


@dataclass
class CacheConfig:
    """Paged cache geometry.  Either ``num_blocks`` is given or it is derived from
    ``kv_cache_memory_gb`` and the bytes one block costs over all cache groups
    (src/tokenvault/config.py:91-102)."""

    block_size: int = 16
    num_blocks: int | None = 256
    kv_cache_memory_gb: float | None = None
    watermark: float = 0.01
    dtype: torch.dtype = torch.float32

    def resolve_num_blocks(self, bytes_per_block: int) -> int:
        if self.num_blocks is not None:
            return int(self.num_blocks)
        if self.kv_cache_memory_gb is None:
            raise ValueError("either num_blocks or kv_cache_memory_gb must be set")
        return max(1, math.floor(self.kv_cache_memory_gb * 1024**3 / max(1, bytes_per_block)))


@dataclass
class SchedulerConfig:
    max_num_seqs: int = 32
    max_num_batched_tokens: int = 2048
    max_model_len: int = 2048
    policy: SchedulingPolicy = SchedulingPolicy.FCFS
    enable_chunked_prefill: bool = True


@dataclass
class EngineConfig:
    cache: CacheConfig = field(default_factory=CacheConfig)
    scheduler: SchedulerConfig = field(default_factory=SchedulerConfig)
    device: str = "cuda"
    dtype: torch.dtype = torch.float32
    seed: int = 0
    # Replay pure-decode steps from captured HIP graphs (fixed-address metadata buffers).
    use_graphs: bool = True
    # When every running request decodes and none waits, the device takes up to this many decode
    # steps by itself (each sampled token becomes the next input there) before the host reads
    # the tokens and looks at stop conditions; 1 makes the host look after every step.
    decode_run_steps: int = 8
    # While such runs follow each other for the same requests, queue the next run on the device
    # before the tokens of the current one are read, so that the device does not wait for the
    # host in between.  A run that turns out not to be wanted (a request stopped, another one
    # arrived) is left unread; what it wrote to the cache is computed again by the next step.
    decode_run_ahead: bool = True

    def __post_init__(self) -> None:
        self.dtype = parse_dtype(self.dtype)
        if self.decode_run_steps < 1:
            raise ValueError("decode_run_steps must be at least 1")
        # The cache holds what the model computes with (src/tokenvault/config.py:150-151).
        self.cache.dtype = self.dtype

    def clamp_to_model(self, max_position_embeddings: int) -> None:
        """``max_model_len = min(max_model_len, max_position_embeddings)``
        (src/tokenvault/config.py:146-149)."""
        self.scheduler.max_model_len = min(self.scheduler.max_model_len, max_position_embeddings)
