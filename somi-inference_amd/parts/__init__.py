"""Parts a layer is put together from, and the registries that name them."""

from .attention import GroupedQueryAttention
from .base import (PAGE, Block, FeedForward, FixedStateSpec, LayerCache, Mixer, Norm, PagedKVSpec, PagedSpec,
                   PageTensor, Part, PartSpec, PositionEncoding, Runtime)
from .block import PreNormBlock
from .embedding import LMHead, TokenEmbedding
from .feed_forward import SwiGLU
from .norm import RMSNorm
from .position import NoPosition, RotaryPosition
from .registry import build_part, part_kinds, register_part, unregister_part
from .residual import ResidualStream

register_part("norm", "rmsnorm", RMSNorm)
register_part("position", "rotary", RotaryPosition)
register_part("position", "none", NoPosition)
register_part("mixer", "gqa_attention", GroupedQueryAttention)
register_part("feed_forward", "swiglu", SwiGLU)
register_part("block", "pre_norm", PreNormBlock)
register_part("embedding", "token_embedding", TokenEmbedding)
register_part("head", "lm_head", LMHead)

__all__ = [
    "Block", "FeedForward", "FixedStateSpec", "GroupedQueryAttention", "LMHead", "LayerCache", "Mixer",
    "NoPosition", "Norm", "PAGE", "PageTensor", "PagedKVSpec", "PagedSpec", "Part", "PartSpec", "PositionEncoding", "PreNormBlock", "RMSNorm",
    "ResidualStream", "RotaryPosition", "Runtime", "SwiGLU", "TokenEmbedding", "build_part", "part_kinds",
    "register_part", "unregister_part",
]
