from tokenmill_amd.parts.attention import GQAttention
from tokenmill_amd.parts.base import (FeedForward, GroupStep, KVCacheSpec, KVCacheView, Mixer, Norm, NormedInput, Part,
                                      PositionEncoding, StateSpec, StateView, StepContext, as_tensor)
from tokenmill_amd.parts.block import PreNormBlock
from tokenmill_amd.parts.embedding import OutputHead, TokenEmbedding
from tokenmill_amd.parts.linear import Linear
from tokenmill_amd.parts.mlp import SwiGLU
from tokenmill_amd.parts.norm import RMSNorm
from tokenmill_amd.parts.position import NoPositionEncoding, RotaryEmbedding

__all__ = ["GQAttention", "FeedForward", "GroupStep", "KVCacheSpec", "KVCacheView", "Mixer", "Norm", "NormedInput", "as_tensor", "Part",
           "PositionEncoding", "StateSpec", "StateView", "StepContext", "PreNormBlock", "OutputHead",
           "TokenEmbedding", "Linear", "SwiGLU", "RMSNorm", "NoPositionEncoding", "RotaryEmbedding"]
