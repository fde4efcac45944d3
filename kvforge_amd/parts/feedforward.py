"""SwiGLU feed-forward: ``down(silu(gate(x)) * up(x))`` (src/tokenvault/model.py:118-132)."""

from __future__ import annotations

import torch

from kvforge_amd.kernels import ops
from kvforge_amd.parts.base import FeedForward, WeightSpec, add_product
from kvforge_amd.registry import register_feed_forward


@register_feed_forward("swiglu")
class SwiGLU(FeedForward):
    replayable = True
    settles_residual = True  # its norm kernel adds what is owed to the stream

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
        # one product for gate and up, rows interleaved: row 2i is gate_i, row 2i+1 is up_i, so
        # a kernel that holds neighbouring output columns holds a whole (gate, up) pair
        self.w_gate_up = torch.stack([g, u], dim=1).reshape(2 * self.inter, self.hidden).contiguous()
        self.w_down = tensors[self._name("down_proj.weight")]
        self.norm_eps = None

    def absorb_norm(self, norm) -> bool:
        if self.norm_eps is not None or not getattr(norm, "foldable_into", lambda m: False)(self.w_gate_up):
            return False
        self.w_gate_up = (self.w_gate_up.float() * norm.weight.float()[None, :]).to(
            torch.bfloat16).contiguous()
        self.norm_eps = norm.eps
        return True

    def kernel_modules(self, dtype: torch.dtype) -> set[str]:
        mods = {"elementwise", "gemm_generic"}
        if dtype == torch.bfloat16:
            mods |= {"gemm_bf16"}
        return mods

    def num_bytes(self) -> int:
        return sum(t.numel() * t.element_size()
                   for t in map(ops.plain_of, (self.w_gate_up, self.w_down)) if t is not None)

    def held_tensors(self) -> list[torch.Tensor]:
        return ops.copies_of(self.w_gate_up) + ops.copies_of(self.w_down)

    def seal(self) -> None:
        self.w_gate_up = ops.streamed(ops.plain_of(self.w_gate_up))
        self.w_down = ops.streamed(ops.plain_of(self.w_down))

    def forward(self, x, step, residual) -> None:
        """``x``: normalised activations, or (after ``absorb_norm``) the fp32 residual stream."""
        n = x.shape[0]
        ws, dt, rms = step.ws, step.act_dtype, self.norm_eps
        act = ws.buf("ffn_act", (n, self.inter), dt)
        if rms is not None and not ops.bf16_kernel_takes(x, self.w_gate_up, True):
            # too many rows for the norm to ride in the projection: a norm kernel of its own,
            # which also adds what the mixer still owes the stream
            normed = ws.buf("normed", (n, self.hidden), dt)
            ops.rmsnorm(x, None, rms, normed, add=step.take_owed(residual))
            x, rms = normed, None
        else:
            step.settle()
        if ops.bf16_kernel_takes(x, self.w_gate_up, rms is not None, True) and self.inter % 2 == 0:
            # one kernel: (norm,) gate/up projection, SwiGLU gate
            ops.gemm_fused(x, self.w_gate_up, act, rms_eps=rms, silu_pairs=True)
        else:
            gu = ws.buf("gate_up", (n, 2 * self.inter), dt)
            ops.gemm(x, self.w_gate_up, gu)
            ops.silu_mul(gu, act, paired=True)
        add_product(step, act, self.w_down, residual)
