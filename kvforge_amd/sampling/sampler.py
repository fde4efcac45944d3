"""Batched token selection on the device (src/tokenvault/sampling.py:40-88): per-row
temperature, top-k, top-p; greedy rows take the argmax.  One kernel launch per batch."""

from __future__ import annotations

from typing import Sequence

import torch

from kvforge_amd.kernels import ops
from kvforge_amd.sampling.params import SamplingParams
from kvforge_amd.sampling.rng import uniform


class Sampler:
    def __init__(self, seed: int = 0, device: torch.device | str = "cuda") -> None:
        self.seed, self.device = int(seed), device

    def __call__(self, logits: torch.Tensor, params: Sequence[SamplingParams],
                 streams: Sequence[int], counters: Sequence[int]) -> list[int]:
        """``logits [R, V]`` fp32; row ``i`` uses ``params[i]`` and the uniform number of
        (seed, ``streams[i]``, ``counters[i]``).  Returns one token id per row."""
        r = logits.shape[0]
        if r == 0:
            return []
        if not (len(params) == len(streams) == len(counters) == r):
            raise ValueError("one SamplingParams, stream and counter per logits row")
        temps = torch.tensor([p.temperature for p in params], dtype=torch.float32)
        us = torch.tensor([0.0 if p.greedy else uniform(self.seed, s, c)
                           for p, s, c in zip(params, streams, counters)], dtype=torch.float32)
        top_k = top_p = None
        if any(p.top_k > 0 for p in params):
            top_k = torch.tensor([p.top_k for p in params], dtype=torch.int32).to(self.device)
        if any(p.top_p < 1.0 for p in params):
            top_p = torch.tensor([p.top_p for p in params], dtype=torch.float32).to(self.device)
        tokens = torch.empty(r, dtype=torch.int32, device=self.device)
        ops.sample(logits, temps.to(self.device), top_k, top_p, us.to(self.device), tokens)
        return tokens.tolist()
