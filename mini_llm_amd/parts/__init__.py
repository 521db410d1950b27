from .attention import CausalSelfAttention
from .base import (
    BLOCKS, FEED_FORWARDS, MIXERS, NORMS, POSITION_ENCODINGS,
    Block, FeedForward, KVNeed, LayerContext, Mixer, Norm, Part, PositionEncoding, StateNeed,
    make_part, register_part,
)
from .block import PreNormBlock
from .embedding import TiedHead, TokenEmbedding
from .feedforward import DenseMLP
from .linear import Linear
from .norms import LayerNorm
from .positions import LearnedPositions

__all__ = [
    "BLOCKS", "FEED_FORWARDS", "MIXERS", "NORMS", "POSITION_ENCODINGS",
    "Block", "FeedForward", "KVNeed", "LayerContext", "Mixer", "Norm", "Part", "PositionEncoding", "StateNeed",
    "make_part", "register_part",
    "CausalSelfAttention", "PreNormBlock", "TiedHead", "TokenEmbedding", "DenseMLP", "Linear", "LayerNorm", "LearnedPositions",
]
