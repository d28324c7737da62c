from .attention import PagedAttention
from .base import (Block, BuildContext, CacheField, CacheSpec, FeedForward, KVCacheSpec, Mixer, Norm, NormFold, Part,
                   Normed, PartialSums, PositionEncoding, Prenormed, StateSpec)
from .block import PreNormBlock
from .embedding import Embedding
from .feed_forward import GatedMLP
from .linear import Linear
from .norm import RMSNorm
from .position import NoPositionEncoding, RotaryHalfSplit

__all__ = [
    "Block", "BuildContext", "CacheField", "CacheSpec", "Embedding", "FeedForward", "GatedMLP", "KVCacheSpec", "Linear", "Mixer",
    "NoPositionEncoding", "Norm", "NormFold", "Normed", "PagedAttention", "Part", "PartialSums", "PositionEncoding", "PreNormBlock", "Prenormed", "RMSNorm",
    "RotaryHalfSplit", "StateSpec",
]
