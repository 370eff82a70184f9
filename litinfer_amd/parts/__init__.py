from .base import (BatchNeeds, Block, FeedForward, Mixer, Norm, PagedKVNeed, PagedNeed, PagedTensor, Part,
                   Runtime, StateNeed, build_part, needs_of, register_part)
from .position import Position, RopeNeox
from .linear import Linear
from .stream import ResidualStream
from .norm import RMSNorm
from .attention import GQAttention
from .mlp import SwiGLUMLP
from .block import PreNormBlock
from .embedding import LinearHead, TokenEmbedding

__all__ = ["BatchNeeds", "Block", "FeedForward", "Mixer", "Norm", "PagedKVNeed", "PagedNeed", "PagedTensor",
           "Part", "Runtime", "StateNeed", "needs_of",
           "build_part", "register_part", "Position", "RopeNeox", "Linear", "ResidualStream", "RMSNorm",
           "GQAttention", "SwiGLUMLP", "PreNormBlock", "LinearHead", "TokenEmbedding"]
