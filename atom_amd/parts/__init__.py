"""Model parts and their registries.  Importing the package registers the built-in parts."""

from .base import (BLOCKS, EMBEDDINGS, FEED_FORWARDS, HEADS, JOINS, MIXERS, NORMS, POSITION_ENCODINGS, Block, Embedding,
                   FeedForward, Head, Join, KVCacheNeed, LatentCacheNeed, Mixer, Norm, ParamSpec, Part, PartChoice,
                   PositionEncoding, Registry, Source, StateNeed)
from . import (attention, block, delta, embedding, experts, join, kv_attention, latent_attention, mlp, norm,  # noqa: F401
               rglru, rope, token_side)
from .attention import GroupedQueryAttention
from .block import PostNormBlock, PreNormBlock, SandwichBlock
from .delta import GatedDeltaRule
from .embedding import BigramEmbedding, LMHead, ScaledEmbedding, TokenEmbedding
from .experts import RoutedExperts
from .join import ConcatProjection
from .kv_attention import KeyValueAttention
from .latent_attention import LatentAttention
from .mlp import GatedMLP
from .norm import LayerNorm, RMSNorm
from .rglru import RealGatedRecurrence
from .rope import BandedRotary, RotaryEncoding, ScaledRotary
from .token_side import TokenSide

__all__ = [
    "BLOCKS", "EMBEDDINGS", "FEED_FORWARDS", "HEADS", "JOINS", "MIXERS", "NORMS", "POSITION_ENCODINGS", "Block",
    "Embedding", "FeedForward", "Head", "Join", "KVCacheNeed", "LatentCacheNeed", "Mixer", "Norm", "ParamSpec", "Part",
    "PartChoice", "PositionEncoding", "Registry", "Source", "StateNeed",
    "GroupedQueryAttention", "PreNormBlock", "LMHead", "TokenEmbedding", "GatedMLP", "RMSNorm", "RotaryEncoding",
    "SandwichBlock", "GatedDeltaRule", "ScaledEmbedding", "RoutedExperts", "ConcatProjection", "LatentAttention",
    "LayerNorm", "ScaledRotary", "PostNormBlock", "BigramEmbedding", "KeyValueAttention", "RealGatedRecurrence",
    "BandedRotary", "TokenSide",
]
