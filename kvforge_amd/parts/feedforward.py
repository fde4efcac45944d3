"""SwiGLU feed-forward: ``down(silu(gate(x)) * up(x))`` (src/tokenvault/model.py:118-132)."""

from __future__ import annotations

import torch

from kvforge_amd.kernels import ops
from kvforge_amd.parts.base import FeedForward, WeightSpec
from kvforge_amd.registry import register_feed_forward


@register_feed_forward("swiglu")
class SwiGLU(FeedForward):
    def __init__(self, prefix: str, hidden: int, intermediate: int) -> None:
        self.prefix, self.hidden, self.inter = prefix, int(hidden), int(intermediate)
        self.w_gate_up: torch.Tensor | None = None
        self.w_down: torch.Tensor | None = None

    def weight_specs(self) -> dict[str, WeightSpec]:
        return {
            self._name("gate_proj.weight"): WeightSpec((self.inter, self.hidden)),
            self._name("up_proj.weight"): WeightSpec((self.inter, self.hidden)),
            self._name("down_proj.weight"): WeightSpec((self.hidden, self.inter)),
        }

    def load(self, tensors: dict[str, torch.Tensor]) -> None:
        g, u = tensors[self._name("gate_proj.weight")], tensors[self._name("up_proj.weight")]
        if g.dtype != u.dtype:
            g, u = g.float(), u.float()
        # one product for gate and up: rows [0, I) are gate, rows [I, 2I) are up
        self.w_gate_up = torch.cat([g, u], dim=0).contiguous()
        self.w_down = tensors[self._name("down_proj.weight")]

    def kernel_modules(self, dtype: torch.dtype) -> set[str]:
        mods = {"elementwise", "gemm_generic"}
        if dtype == torch.bfloat16:
            mods |= {"gemm_bf16"}
        return mods

    def num_bytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in (self.w_gate_up, self.w_down)
                   if t is not None)

    def forward(self, x, step, residual) -> None:
        n = x.shape[0]
        gu = step.ws.buf("gate_up", (n, 2 * self.inter), x.dtype)
        ops.gemm(x, self.w_gate_up, gu)
        act = step.ws.buf("ffn_act", (n, self.inter), x.dtype)
        ops.silu_mul(gu, act)
        ops.gemm(act, self.w_down, residual, accumulate=True)
