from kvforge_amd.parts.base import (Block, CacheSpec, FeedForward, LayerCall, LayerState, Mixer,
                                    ModelSpec, Norm, Part, Positions, StateSpec, WeightSpec)
from kvforge_amd.parts.norm import RMSNorm
from kvforge_amd.parts.positions import RotaryPositions, scaled_inv_freq
from kvforge_amd.parts.attention import PagedAttention
from kvforge_amd.parts.feedforward import SwiGLU
from kvforge_amd.parts.embedding import LMHead, TokenEmbedding
from kvforge_amd.parts.block import PreNormBlock

__all__ = ["Block", "CacheSpec", "FeedForward", "LayerCall", "LayerState", "Mixer", "ModelSpec",
           "Norm", "Part", "Positions", "StateSpec", "WeightSpec", "RMSNorm", "RotaryPositions",
           "scaled_inv_freq", "PagedAttention", "SwiGLU", "LMHead", "TokenEmbedding",
           "PreNormBlock"]
