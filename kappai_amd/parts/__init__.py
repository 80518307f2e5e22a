from .attention import GroupedQueryAttention
from .base import (BLOCKS, FEED_FORWARDS, MIXERS, NORMS, POSITION_ENCODINGS, Block, FeedForward,
                   Hidden, Mixer, Norm, Part, PositionEncoding, make_part, register_part)
from .block import PreNormBlock
from .embedding import OutputHead, TokenEmbedding
from .feed_forward import SwiGLU
from .linear import Linear
from .norm import RMSNorm
from .rotary import RotaryEncoding, Rotation
from .shortconv import GatedShortConv

__all__ = ["GroupedQueryAttention", "BLOCKS", "FEED_FORWARDS", "MIXERS", "NORMS",
           "POSITION_ENCODINGS", "Block", "FeedForward", "Hidden", "Mixer", "Norm", "Part",
           "PositionEncoding", "make_part", "register_part", "PreNormBlock", "OutputHead",
           "TokenEmbedding", "SwiGLU", "Linear", "RMSNorm", "RotaryEncoding", "Rotation",
           "GatedShortConv"]
