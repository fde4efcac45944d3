"""Rotary position encoding: fp32 cos/sin tables that attention applies to queries and keys.

Angles follow src/tokenvault/model.py:41-50: ``inv_freq[j] = 1 / theta^(2j/d)`` in fp32,
``angle = float(position) * inv_freq`` in fp32, then cos and sin.  The tables are computed once
on the host with exactly these operations, so the kernels never evaluate a trigonometric
function of a large angle themselves.  Frequency scaling of type ``llama3`` (absent from the
reference) rescales ``inv_freq`` before the tables are made.
"""

from __future__ import annotations

import math

import torch

from kvforge_amd.config.model import RopeScaling
from kvforge_amd.parts.base import Positions
from kvforge_amd.registry import register_positions


def scaled_inv_freq(rot_dim: int, theta: float, scaling: RopeScaling | None) -> torch.Tensor:
    inv_freq = 1.0 / (theta ** (torch.arange(0, rot_dim, 2, dtype=torch.float32) / rot_dim))
    if scaling is None:
        return inv_freq
    if scaling.rope_type != "llama3":
        raise ValueError(f"unsupported rope scaling {scaling.rope_type!r}")
    f = inv_freq.double()
    orig = float(scaling.original_max_position_embeddings)
    wavelen = 2.0 * math.pi / f
    low_wavelen = orig / scaling.low_freq_factor
    high_wavelen = orig / scaling.high_freq_factor
    smooth = (orig / wavelen - scaling.low_freq_factor) / (
        scaling.high_freq_factor - scaling.low_freq_factor)
    blended = (1.0 - smooth) * f / scaling.factor + smooth * f
    out = torch.where(wavelen < high_wavelen, f,
                      torch.where(wavelen > low_wavelen, f / scaling.factor, blended))
    return out.float()


@register_positions("rotary")
class RotaryPositions(Positions):
    """Half-split rotary pairs (element ``i`` with ``i + rot_dim/2``) over the first ``rot_dim``
    elements of each head."""

    replayable = True

    def __init__(self, rot_dim: int, theta: float, scaling: RopeScaling | None = None) -> None:
        if rot_dim <= 0 or rot_dim % 2:
            raise ValueError(f"rotary width must be positive and even, got {rot_dim}")
        self.rot_dim, self.theta, self.scaling = int(rot_dim), float(theta), scaling
        self.inv_freq = scaled_inv_freq(self.rot_dim, self.theta, scaling)
        self.cos: torch.Tensor | None = None
        self.sin: torch.Tensor | None = None

    def prepare(self, max_positions: int, device: torch.device | str) -> None:
        pos = torch.arange(int(max_positions), dtype=torch.int64)
        freqs = pos.float()[:, None] * self.inv_freq.float()
        self.cos = freqs.cos().contiguous().to(device)
        self.sin = freqs.sin().contiguous().to(device)

    def kernel_modules(self, dtype: torch.dtype) -> set[str]:
        return {"elementwise"}
