"""Batched token selection on the device (src/tokenvault/sampling.py:40-88): per-row
temperature, top-k, top-p; greedy rows take the argmax.  One kernel launch per batch; the rows'
parameters travel in one copy from a pinned staging buffer that is kept across calls."""

from __future__ import annotations

from typing import Sequence

import torch

from kvforge_amd.kernels import ops
from kvforge_amd.sampling.params import SamplingParams
from kvforge_amd.sampling.rng import uniform


class Sampler:
    def __init__(self, seed: int = 0, device: torch.device | str = "cuda") -> None:
        self.seed, self.device = int(seed), device
        self._rows = 0
        self._host = self._dev = self._tokens = None

    def _buffers(self, rows: int):
        """Four values per row (temperature, uniform number, top-p, top-k as a float's bits)."""
        if rows > self._rows:
            self._rows = max(rows, 2 * self._rows, 64)
            pinned = torch.device(self.device).type == "cuda"
            self._host = torch.zeros(4, self._rows, dtype=torch.float32, pin_memory=pinned)
            self._dev = torch.zeros(4, self._rows, dtype=torch.float32, device=self.device)
            self._tokens = torch.zeros(self._rows, dtype=torch.int32, device=self.device)
        return self._host, self._dev, self._tokens

    def __call__(self, logits: torch.Tensor, params: Sequence[SamplingParams],
                 streams: Sequence[int], counters: Sequence[int]) -> list[int]:
        """``logits [R, V]`` fp32; row ``i`` uses ``params[i]`` and the uniform number of
        (seed, ``streams[i]``, ``counters[i]``).  Returns one token id per row."""
        r = logits.shape[0]
        if r == 0:
            return []
        if not (len(params) == len(streams) == len(counters) == r):
            raise ValueError("one SamplingParams, stream and counter per logits row")
        host, dev, tokens = self._buffers(r)
        host[0, :r] = torch.tensor([p.temperature for p in params], dtype=torch.float32)
        host[1, :r] = torch.tensor([0.0 if p.greedy else uniform(self.seed, s, c)
                                    for p, s, c in zip(params, streams, counters)], dtype=torch.float32)
        host[2, :r] = torch.tensor([p.top_p for p in params], dtype=torch.float32)
        host[3, :r].view(torch.int32)[:] = torch.tensor([p.top_k for p in params], dtype=torch.int32)
        dev.copy_(host, non_blocking=True)       # the whole (small) buffer: one contiguous copy
        top_k = dev[3, :r].view(torch.int32) if any(p.top_k > 0 for p in params) else None
        top_p = dev[2, :r] if any(p.top_p < 1.0 for p in params) else None
        ops.sample(logits, dev[0, :r], top_k, top_p, dev[1, :r], tokens[:r])
        return tokens[:r].tolist()      # waits for the device: the staging buffer is free again
