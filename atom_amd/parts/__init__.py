"""Model parts and their registries.  Importing the package registers the built-in parts."""

from .base import (BLOCKS, EMBEDDINGS, FEED_FORWARDS, HEADS, JOINS, MIXERS, NORMS, POSITION_ENCODINGS, Block, Embedding,
                   FeedForward, Head, Join, KVCacheNeed, LatentCacheNeed, Mixer, Norm, ParamSpec, Part, PartChoice,
                   PositionEncoding, Registry, Source, StateNeed)
from . import (attention, block, delta, embedding, experts, join, kv_attention, latent_attention, mlp, norm,  # noqa: F401
               parallel, plain_attention, rglru, rope, shift, state_space, time_mix, together_attention, token_side)
from .attention import GroupedQueryAttention
from .block import NormedSumBlock, PostNormBlock, PreNormBlock, SandwichBlock
from .delta import GatedDeltaRule
from .embedding import BigramEmbedding, LMHead, PositionedEmbedding, ScaledEmbedding, TokenEmbedding
from .experts import RoutedExperts
from .join import AddFirst, ConcatProjection
from .kv_attention import KeyValueAttention
from .latent_attention import LatentAttention
from .mlp import DenseMLP, GatedMLP
from .norm import LayerNorm, RMSNorm
from .parallel import JointNeed, ParallelMixer
from .plain_attention import PlainAttention
from .rglru import RealGatedRecurrence
from .rope import BandedRotary, HalfRotary, RotaryEncoding, ScaledRotary
from .shift import ShiftedMixer
from .together_attention import TogetherAttention
from .state_space import StateSpaceMixer
from .time_mix import TimeMixRecurrence
from .token_side import TokenSide

__all__ = [
    "BLOCKS", "EMBEDDINGS", "FEED_FORWARDS", "HEADS", "JOINS", "MIXERS", "NORMS", "POSITION_ENCODINGS", "Block",
    "Embedding", "FeedForward", "Head", "Join", "KVCacheNeed", "LatentCacheNeed", "Mixer", "Norm", "ParamSpec", "Part",
    "PartChoice", "PositionEncoding", "Registry", "Source", "StateNeed",
    "GroupedQueryAttention", "PreNormBlock", "LMHead", "TokenEmbedding", "GatedMLP", "RMSNorm", "RotaryEncoding",
    "SandwichBlock", "GatedDeltaRule", "ScaledEmbedding", "RoutedExperts", "ConcatProjection", "LatentAttention",
    "LayerNorm", "ScaledRotary", "PostNormBlock", "BigramEmbedding", "KeyValueAttention", "RealGatedRecurrence",
    "BandedRotary", "TokenSide", "AddFirst", "DenseMLP", "JointNeed", "ParallelMixer", "PlainAttention",
    "PositionedEmbedding", "StateSpaceMixer", "TimeMixRecurrence", "NormedSumBlock", "HalfRotary", "ShiftedMixer",
    "TogetherAttention",
]
