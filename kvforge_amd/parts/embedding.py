"""Token embedding and the output head (src/tokenvault/model.py:153-158,169-170,190-191)."""

from __future__ import annotations

import torch

from kvforge_amd.kernels import ops
from kvforge_amd.parts.base import Embedding, Head, WeightSpec


class TokenEmbedding(Embedding):
    """``h0 = table[ids]`` into the fp32 residual stream; no scaling."""

    replayable = True

    def __init__(self, prefix: str, vocab: int, hidden: int) -> None:
        self.prefix, self.vocab, self.hidden = prefix, int(vocab), int(hidden)
        self.table: torch.Tensor | None = None

    def weight_specs(self) -> dict[str, WeightSpec]:
        return {self._name("weight"): WeightSpec((self.vocab, self.hidden))}

    def load(self, tensors: dict[str, torch.Tensor]) -> None:
        self.table = tensors[self._name("weight")]

    def kernel_modules(self, dtype: torch.dtype) -> set[str]:
        return {"elementwise"}

    def held_tensors(self) -> list[torch.Tensor]:
        return [] if self.table is None else [self.table]

    def forward(self, ids: torch.Tensor, out: torch.Tensor) -> None:
        ops.embed(ids, self.table, out)

    def pick_table(self) -> torch.Tensor | None:
        t = self.table
        return t if t is not None and t.dtype == torch.bfloat16 else None


class LMHead(Head):
    """``logits = x @ W^T`` in fp32 output.  ``tied_to``: the checkpoint name of the embedding
    table when the head shares it (then no tensor of its own is expected)."""

    replayable = True

    def __init__(self, prefix: str, vocab: int, hidden: int, tied_to: str | None = None) -> None:
        self.prefix, self.vocab, self.hidden, self.tied_to = prefix, int(vocab), int(hidden), tied_to
        self.weight: torch.Tensor | None = None

    def weight_specs(self) -> dict[str, WeightSpec]:
        if self.tied_to is not None:
            return {self.tied_to: WeightSpec((self.vocab, self.hidden))}
        return {self._name("weight"): WeightSpec((self.vocab, self.hidden))}

    def load(self, tensors: dict[str, torch.Tensor]) -> None:
        self.weight = tensors[self.tied_to if self.tied_to is not None else self._name("weight")]

    def kernel_modules(self, dtype: torch.dtype) -> set[str]:
        return {"gemm_generic"} | ({"gemm_bf16"} if dtype == torch.bfloat16 else set())

    def num_bytes(self) -> int:
        w = ops.plain_of(self.weight)
        return w.numel() * w.element_size() if w is not None else 0

    def held_tensors(self) -> list[torch.Tensor]:
        return ops.copies_of(self.weight)

    def seal(self) -> None:
        # a tied table stays as it is for the embedding; the head streams a tiled copy
        self.weight = ops.streamed(ops.plain_of(self.weight))

    def forward(self, x: torch.Tensor, logits: torch.Tensor) -> None:
        ops.gemm(x, self.weight, logits)

    def can_pick(self, rows: int) -> bool:
        """Whether ``pick`` takes so many rows with this weight."""
        return (isinstance(self.weight, ops.StreamedWeight) and 0 < rows <= ops.FUSED_NORM_MAX_M
                and self.hidden % 8 == 0)

    def pick(self, x: torch.Tensor, residual: torch.Tensor, step, tail) -> None:
        """The tail of a greedy decode step in one kernel (``ops.gemm_pick``): ``x`` holds the
        normalised row of every sequence, all of them wanted."""
        ops.gemm_pick(x, self.weight, residual, tail.tokens, step.token_ids, step.positions,
                      step.ctx_lens, tail.ring, tail.run_counter, tail.embed_table, tail.work)
