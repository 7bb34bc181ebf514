"""Parts that models are built from."""
from .base import (Block, CacheNeeds, FeedForward, HalfSplitRotation, KVSpec, Mixer, Norm, Part, PositionEncoding,
                   Runtime, StateSpec, WeightSpec, create_part, register_part, registered_parts)
from .norm import RMSNorm
from .position import NoPosition, Rotary
from .attention import Attention
from .feedforward import GatedMLP
from .block import PreNormBlock
from .embedding import Embedding, OutputHead

__all__ = [
    "Block", "CacheNeeds", "FeedForward", "HalfSplitRotation", "KVSpec", "Mixer", "Norm", "Part", "PositionEncoding",
    "Runtime", "StateSpec", "WeightSpec", "create_part", "register_part", "registered_parts",
    "RMSNorm", "NoPosition", "Rotary", "Attention", "GatedMLP", "PreNormBlock", "Embedding", "OutputHead",
]
