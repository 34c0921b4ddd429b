"""Model parts and their registries.  Importing the package registers the built-in parts."""

from .base import (BLOCKS, EMBEDDINGS, FEED_FORWARDS, HEADS, MIXERS, NORMS, POSITION_ENCODINGS, Block, Embedding,
                   FeedForward, Head, KVCacheNeed, Mixer, Norm, ParamSpec, Part, PartChoice, PositionEncoding, Registry,
                   Source, StateNeed)
from . import attention, block, embedding, mlp, norm, rope  # noqa: F401  (registration)
from .attention import GroupedQueryAttention
from .block import PreNormBlock
from .embedding import LMHead, TokenEmbedding
from .mlp import GatedMLP
from .norm import RMSNorm
from .rope import RotaryEncoding

__all__ = [
    "BLOCKS", "EMBEDDINGS", "FEED_FORWARDS", "HEADS", "MIXERS", "NORMS", "POSITION_ENCODINGS", "Block", "Embedding",
    "FeedForward", "Head", "KVCacheNeed", "Mixer", "Norm", "ParamSpec", "Part", "PartChoice", "PositionEncoding",
    "Registry", "Source", "StateNeed",
    "GroupedQueryAttention", "PreNormBlock", "LMHead", "TokenEmbedding", "GatedMLP", "RMSNorm", "RotaryEncoding",
]
