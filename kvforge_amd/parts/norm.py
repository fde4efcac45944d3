"""RMS norm over the fp32 residual stream (src/tokenvault/model.py:28-38)."""

from __future__ import annotations

import torch

from kvforge_amd.kernels import ops
from kvforge_amd.parts.base import Norm, WeightSpec
from kvforge_amd.registry import register_norm


@register_norm("rmsnorm")
class RMSNorm(Norm):
    """``y = x * rsqrt(mean(x^2) + eps) * weight`` in fp32, rounded once to the output type."""

    replayable = True

    def __init__(self, prefix: str, width: int, eps: float) -> None:
        self.prefix, self.width, self.eps = prefix, int(width), float(eps)
        self.weight: torch.Tensor | None = None

    def weight_specs(self) -> dict[str, WeightSpec]:
        return {self._name("weight"): WeightSpec((self.width,), init="norm", std=0.1)}

    def load(self, tensors: dict[str, torch.Tensor]) -> None:
        self.weight = tensors[self._name("weight")]

    def kernel_modules(self, dtype: torch.dtype) -> set[str]:
        return {"elementwise"}

    def num_bytes(self) -> int:
        return self.weight.numel() * self.weight.element_size() if self.weight is not None else 0

    def held_tensors(self) -> list[torch.Tensor]:
        return [] if self.weight is None else [self.weight]

    def forward(self, x: torch.Tensor, out: torch.Tensor, rows: torch.Tensor | None = None,
                add: torch.Tensor | None = None) -> None:
        ops.rmsnorm(x, self.weight, self.eps, out, rows, add)

    def foldable_into(self, matrix: torch.Tensor) -> bool:
        """Whether this norm's weight may be multiplied into the columns of a bf16 matrix: only
        when it is itself held in bf16 (a weight stored in 32-bit stays a 32-bit multiply)."""
        return (self.weight is not None and self.weight.dtype == torch.bfloat16
                and matrix.dtype == torch.bfloat16 and matrix.shape[1] == self.width)
