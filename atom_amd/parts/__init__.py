"""Model parts and their registries.  Importing the package registers the built-in parts."""

from .base import (BLOCKS, EMBEDDINGS, FEED_FORWARDS, HEADS, JOINS, MIXERS, NORMS, POSITION_ENCODINGS, Block, Embedding,
                   FeedForward, Head, Join, KVCacheNeed, LatentCacheNeed, Mixer, Norm, ParamSpec, Part, PartChoice,
                   PositionEncoding, Registry, Source, StateNeed)
from . import attention, block, delta, embedding, experts, join, latent_attention, mlp, norm, rope  # noqa: F401  (registration)
from .attention import GroupedQueryAttention
from .block import PreNormBlock, SandwichBlock
from .delta import GatedDeltaRule
from .embedding import LMHead, ScaledEmbedding, TokenEmbedding
from .experts import RoutedExperts
from .join import ConcatProjection
from .latent_attention import LatentAttention
from .mlp import GatedMLP
from .norm import LayerNorm, RMSNorm
from .rope import RotaryEncoding, ScaledRotary

__all__ = [
    "BLOCKS", "EMBEDDINGS", "FEED_FORWARDS", "HEADS", "JOINS", "MIXERS", "NORMS", "POSITION_ENCODINGS", "Block",
    "Embedding", "FeedForward", "Head", "Join", "KVCacheNeed", "LatentCacheNeed", "Mixer", "Norm", "ParamSpec", "Part",
    "PartChoice", "PositionEncoding", "Registry", "Source", "StateNeed",
    "GroupedQueryAttention", "PreNormBlock", "LMHead", "TokenEmbedding", "GatedMLP", "RMSNorm", "RotaryEncoding",
    "SandwichBlock", "GatedDeltaRule", "ScaledEmbedding", "RoutedExperts", "ConcatProjection", "LatentAttention",
    "LayerNorm", "ScaledRotary",
]
