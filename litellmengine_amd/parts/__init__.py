from .attention import ConvAttention, PagedAttention, SinkAttention
from .base import (Block, BuildContext, CacheField, Carried, CacheSpec, FeedForward, KVCacheSpec, Mixer, Norm, NormFold, Part,
                   Normed, PartialSums, PositionEncoding, Prenormed, ScaledSum, StateSpec)
from .block import ParallelBlock, PostNormBlock, PreNormBlock, SandwichBlock
from .delta import GatedDeltaMixer
from .embedding import Embedding
from .feed_forward import GatedMLP, PlainMLP
from .latent_attention import LatentAttention
from .linear import Linear
from .moe import GroupLimitedMLP, RoutedMLP, ScoreRoutedMLP
from .norm import RMSNorm
from .position import NoPositionEncoding, RotaryHalfSplit, RotaryInterleaved
from .recurrent import MinGRU
from .side_by_side import SideBySideMixer
from .wkv import WKVMixer

__all__ = [
    "Block", "BuildContext", "CacheField", "CacheSpec", "Carried", "LatentAttention", "MinGRU", "PostNormBlock",
    "RoutedMLP", "RotaryInterleaved", "Embedding", "FeedForward", "GatedMLP", "KVCacheSpec", "Linear", "Mixer",
    "NoPositionEncoding", "Norm", "NormFold", "Normed", "PagedAttention", "Part", "PartialSums", "PositionEncoding", "PreNormBlock", "Prenormed", "RMSNorm",
    "RotaryHalfSplit", "StateSpec", "GroupLimitedMLP", "ParallelBlock", "ScaledSum", "SinkAttention", "WKVMixer",
    "ConvAttention", "SandwichBlock", "PlainMLP", "ScoreRoutedMLP", "SideBySideMixer", "GatedDeltaMixer",
]
