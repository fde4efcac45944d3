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

    def parts(self) -> list[Part]:
        return [self.mixer_norm, self.mixer, self.ffn_norm, self.ffn]

    def forward(self, residual, step, layer: LayerState) -> None:
        x = step.ws.buf("normed", tuple(residual.shape), step.act_dtype)
        self.mixer_norm.forward(residual, x)
        self.mixer.forward(x, step, layer, residual)
        self.ffn_norm.forward(residual, x)
        self.ffn.forward(x, step, residual)
