"""The step function: a batch of (request, its next tokens), portions of prompts beside single
decoded tokens, cut anywhere, run as one batch from the cache; logits come back for the wanted
places.  The counterpart of the reference's ``ModelRunner.execute``
(src/tokenvault/batching/continuous.py:90-117).

Preconditions, as in the reference: the request's block tables already cover
``start_pos + len(tokens)`` (the scheduler or the replay program asked the cache manager), and
positions below ``start_pos`` are in the cache.
"""

from __future__ import annotations

from typing import Sequence

import torch

from kvforge_amd.cache.manager import CacheManager
from kvforge_amd.cache.storage import PagedStorage, StateStorage, bytes_per_block
from kvforge_amd.engine.batch import MetaBuffers, Step, StepEntry, Workspace, fill_step
from kvforge_amd.kernels import library
from kvforge_amd.models.transformer import Transformer


class ModelRunner:
    def __init__(self, model: Transformer, block_size: int, num_blocks: "int | list[int]",
                 max_num_seqs: int, max_num_batched_tokens: int, max_model_len: int,
                 watermark: float = 0.0) -> None:
        if torch.device(model.device).type != "cuda":
            raise RuntimeError("the engine runs on the GPU only; there is no CPU path")
        if not torch.cuda.is_available():
            raise RuntimeError("no GPU is visible to this process")
        library.ensure(model.kernel_modules())
        self.model = model
        self.device = model.device
        self.block_size = int(block_size)
        self.max_model_len = int(max_model_len)
        groups = model.cache_groups
        counts = [num_blocks] * len(groups) if isinstance(num_blocks, int) else list(num_blocks)
        self.cache = CacheManager(block_size, groups, counts,
                                  num_state_slots=max_num_seqs if model.state_specs else 0,
                                  watermark=watermark)
        self.storage = PagedStorage(groups, counts, block_size, model.dtype, self.device)
        self.states = StateStorage(model.state_specs, max_num_seqs, self.device)
        model.attach(self.storage, self.states)
        model.prepare(self.max_model_len)
        width = -(-self.max_model_len // self.block_size)
        self.meta = MetaBuffers(max(max_num_batched_tokens, max_num_seqs), max_num_seqs,
                                [width] * len(groups), self.device)
        self.ws = Workspace(self.device)
        self.num_forward_passes = 0
        self.num_tokens_processed = 0

    @staticmethod
    def bytes_per_block(model: Transformer, block_size: int) -> int:
        return bytes_per_block(model.cache_groups, block_size, model.dtype)

    def _slot_of(self, request_id: str) -> int:
        return self.cache.slots.slot(request_id) if self.cache.slots.num_slots else -1

    def build_step(self, entries: Sequence[StepEntry], pad_to: int | None = None
                   ) -> tuple[Step, list[int]]:
        for e in entries:
            if e.start_pos + len(e.token_ids) > self.max_model_len:
                raise ValueError(f"request {e.request_id} would pass max_model_len "
                                 f"{self.max_model_len}")
        step = Step()
        step.ws, step.act_dtype, step.device = self.ws, self.model.dtype, self.device
        counts = fill_step(step, self.meta, entries, self.cache.block_table, self._slot_of,
                           self.block_size, pad_to)
        return step, counts

    @torch.inference_mode()
    def step(self, entries: Sequence[StepEntry]) -> torch.Tensor:
        """One forward over the entries; fp32 logits ``[sum of wanted places, vocab]``, rows in
        entry order then place order.  The tensor is a view of memory the next step reuses."""
        step, _ = self.build_step(entries)
        logits = self.model.forward(step)
        self.num_forward_passes += 1
        self.num_tokens_processed += step.n_tokens
        return logits

    @torch.inference_mode()
    def step_and_sample(self, entries: Sequence[StepEntry], sampler, params, streams, counters
                        ) -> list[int]:
        """One forward, then one token for every wanted place (in row order)."""
        logits = self.step(entries)
        if logits.shape[0] != len(params):
            raise ValueError("one SamplingParams per wanted place")
        return sampler(logits, params, streams, counters)
