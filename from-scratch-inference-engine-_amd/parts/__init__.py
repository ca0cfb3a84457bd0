"""Parts that layers are put together from: mixers, feed-forwards, norms, position encodings,
and the arrangement of a block."""

from .base import (Block, FeedForward, HiddenState, Mixer, Norm, ParamDecl, Part, PositionEncoding,
                   known_parts, make_part, prepare_parts, register_part)
from .attention import AttentionPlanner, GQAttention
from .block import PreNormBlock
from .embedding import LMHead, TokenEmbedding
from .linear import Linear
from .mlp import SwiGLU
from .norm import RMSNorm
from .rope import NoPositionEncoding, RotaryEncoding

__all__ = ["AttentionPlanner", "Block", "FeedForward", "GQAttention", "HiddenState", "LMHead",
           "Linear", "Mixer", "NoPositionEncoding", "Norm", "ParamDecl", "Part", "PositionEncoding",
           "PreNormBlock", "RMSNorm", "RotaryEncoding", "SwiGLU", "TokenEmbedding", "known_parts",
           "make_part", "prepare_parts", "register_part"]
