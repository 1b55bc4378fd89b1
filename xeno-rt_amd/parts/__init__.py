"""Parts that models are built from."""
from .base import (Block, CacheNeeds, FeedForward, HalfSplitRotation, KVSpec, Mixer, Norm, Part, PositionEncoding,
                   Runtime, StateSpec, WeightSpec, create_part, register_part, registered_parts)
from .norm import LayerNorm, OffsetRMSNorm, RMSNorm, ScalarRMSNorm
from .position import DistanceBuckets, DistanceSlopes, NoPosition, PairRotation, Rotary
from .convolution import ShortConvolution, TokenShift
from .attention import Attention, SharedValues
from .latent import LatentAttention
from .recurrent import GatedLinearAttention, LightningAttention, Retention, SelectiveStateSpace, StateSpaceDuality, TimeMixWKV
from .parallel import ParallelMixer, WeightedPair
from .feedforward import ClampedGLU, DenseMLP, ExpertsMLP, GatedMLP
from .block import HyperConnectionBlock, ParallelBlock, PreNormBlock, ResidualStreams, SandwichBlock
from .embedding import Embedding, HashedPairEmbedding, OutputHead, PositionedEmbedding, TokenSideInput, TokenSideTable

__all__ = [
    "Block", "CacheNeeds", "FeedForward", "HalfSplitRotation", "KVSpec", "Mixer", "Norm", "Part", "PositionEncoding",
    "Runtime", "StateSpec", "WeightSpec", "create_part", "register_part", "registered_parts",
    "RMSNorm", "NoPosition", "Rotary", "Attention", "GatedMLP", "PreNormBlock", "Embedding", "OutputHead",
    "ScalarRMSNorm", "DistanceSlopes", "ShortConvolution", "TokenShift", "GatedLinearAttention", "Retention", "TimeMixWKV",
    "ParallelMixer", "DenseMLP", "PositionedEmbedding", "LayerNorm", "DistanceBuckets", "PairRotation", "SharedValues",
    "SandwichBlock", "OffsetRMSNorm", "SelectiveStateSpace", "StateSpaceDuality", "WeightedPair", "ClampedGLU", "ExpertsMLP",
    "ParallelBlock", "HashedPairEmbedding", "TokenSideInput", "TokenSideTable", "HyperConnectionBlock", "ResidualStreams",
    "LatentAttention", "LightningAttention",
]
