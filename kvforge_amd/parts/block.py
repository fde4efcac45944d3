"""Pre-norm residual block: ``h += mixer(norm1(h)); h += ffn(norm2(h))``
(src/tokenvault/model.py:135-143,185-187).  The residual stream is fp32 in every mode; the
mixer's and the feed-forward's last products add into it."""

from __future__ import annotations

from kvforge_amd.parts.base import Block, FeedForward, LayerState, Mixer, Norm, Part
from kvforge_amd.registry import register_block


@register_block("pre_norm")
class PreNormBlock(Block):
    def __init__(self, mixer_norm: Norm, mixer: Mixer, ffn_norm: Norm, ffn: FeedForward) -> None:
        self.mixer_norm, self.mixer, self.ffn_norm, self.ffn = mixer_norm, mixer, ffn_norm, ffn

        self.mixer_takes_residual = self.ffn_takes_residual = False

    def parts(self) -> list[Part]:
        return [self.mixer_norm, self.mixer, self.ffn_norm, self.ffn]

    def load(self, tensors) -> None:
        super().load(tensors)
        # a part may apply the norm in front of it inside its own first kernel
        self.mixer_takes_residual = self.mixer.absorb_norm(self.mixer_norm)
        self.ffn_takes_residual = self.ffn.absorb_norm(self.ffn_norm)

    def forward(self, residual, step, layer: LayerState) -> None:
        if self.mixer_takes_residual:
            if not self.mixer.settles_residual:
                step.settle()
            self.mixer.forward(residual, step, layer, residual)
        else:
            x = step.ws.buf("normed", tuple(residual.shape), step.act_dtype)
            self.mixer_norm.forward(residual, x, add=step.take_owed(residual))
            self.mixer.forward(x, step, layer, residual)
        if self.ffn_takes_residual:
            if not self.ffn.settles_residual:
                step.settle()
            self.ffn.forward(residual, step, residual)
        else:
            x = step.ws.buf("normed", tuple(residual.shape), step.act_dtype)
            self.ffn_norm.forward(residual, x, add=step.take_owed(residual))
            self.ffn.forward(x, step, residual)
