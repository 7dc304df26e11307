from .attention import Attention
from .base import (Block, CacheBinding, FeedForward, KVRequest, Mixer, Norm, Part, PositionEncoding,
                   Runtime, StateRequest, StepArrays, StepContext, Workspace)
from .block import PreNormBlock
from .embedding import LMHead, TokenEmbedding
from .feedforward import SwiGLU
from .linear import Linear
from .norm import RMSNorm
from .position import NoPosition, RotaryEmbedding, rotary_inv_freq

__all__ = ["Attention", "Block", "CacheBinding", "FeedForward", "KVRequest", "Mixer", "Norm", "Part",
           "PositionEncoding", "Runtime", "StateRequest", "StepArrays", "StepContext", "Workspace", "PreNormBlock",
           "LMHead", "TokenEmbedding", "SwiGLU", "Linear", "RMSNorm", "NoPosition", "RotaryEmbedding",
           "rotary_inv_freq"]
