from kvforge_amd.parts.base import (BLOCK, Block, CacheSpec, Embedding, FeedForward, Head, LayerCall,
                                    LayerState, Mixer, ModelSpec, Norm, PageTensor, Part, Positions, StateSpec,
                                    WeightSpec, attention_pages)
from kvforge_amd.parts.norm import RMSNorm
from kvforge_amd.parts.positions import RotaryPositions, scaled_inv_freq
from kvforge_amd.parts.attention import PagedAttention
from kvforge_amd.parts.feedforward import SwiGLU
from kvforge_amd.parts.embedding import LMHead, TokenEmbedding
from kvforge_amd.parts.block import PreNormBlock

__all__ = ["BLOCK", "PageTensor", "attention_pages", "Block", "CacheSpec", "Embedding", "FeedForward", "Head", "LayerCall", "LayerState", "Mixer", "ModelSpec",
           "Norm", "Part", "Positions", "StateSpec", "WeightSpec", "RMSNorm", "RotaryPositions",
           "scaled_inv_freq", "PagedAttention", "SwiGLU", "LMHead", "TokenEmbedding",
           "PreNormBlock"]
