"""The parts a layer is put together from, and the registries of their kinds."""
from .base import (Block, CacheSpec, FeedForward, Mixer, Norm, Part, PositionEncoding, StateSpec, WeightSpec,
                   make_part, register_block, register_feed_forward, register_mixer, register_norm,
                   register_position, registered_kinds)
from .attention import PagedAttention
from .block import PreNormBlock
from .embedding import OutputHead, TokenEmbedding
from .feed_forward import SwiGLU
from .linear import linear
from .norm import RMSNorm
from .position import NoPosition, RotaryEncoding

__all__ = ["Block", "CacheSpec", "FeedForward", "Mixer", "Norm", "Part", "PositionEncoding", "StateSpec",
           "WeightSpec", "make_part", "register_block", "register_feed_forward", "register_mixer", "register_norm",
           "register_position", "registered_kinds", "PagedAttention", "PreNormBlock", "OutputHead",
           "TokenEmbedding", "SwiGLU", "linear", "RMSNorm", "NoPosition", "RotaryEncoding"]
