from .attention import AttentionNames, AttentionPlan, AttentionTuning, GQAttention, TileLaunchCost, build_attention_plan, group_tiling
from .base import (INT_TABLE, MATRIX, VECTOR, Block, FeedForward, Mixer, Norm, PagedAndStateSpec, PagedKVSpec, ParamSpec, Part,
                   PositionEncoding, StateSpec)
from .block import DepthAverage, HyperConnection, MultiStreamBlock, ParallelGatedBlock, PostNormBlock, PreNormBlock, SandwichBlock
from .conv import ShortConvolution
from .delta import GatedDeltaNames, GatedDeltaRule
from .differential import DifferentialAttention, DifferentialNames
from .embedding import NormedTokenEmbedding, TokenEmbedding
from .experts import RoutedExperts
from .kernel_namespace import KernelNamespace
from .latent_attention import LatentAttention, LatentAttentionNames
from .linear import Linear
from .mlp import GatedMLP, GatedMLPNames, PlainMLP
from .norm import RMSNorm, StreamReadNorm
from .parallel import ParallelMixers, ScaledPair
from .recurrent import (GatedLinearAttention, GatedLinearAttentionNames, MatrixMemory, MatrixMemoryNames, TimeMixing, TimeMixingNames,
                        TokenShift)
from .rope import NoPosition, PairedRotaryPosition, RotaryPosition

__all__ = ["KernelNamespace", "AttentionNames", "AttentionTuning", "TileLaunchCost", "GatedMLPNames", "AttentionPlan", "GQAttention", "build_attention_plan", "group_tiling", "INT_TABLE", "MATRIX", "VECTOR",
           "Block", "FeedForward", "Mixer", "Norm", "PagedKVSpec", "ParamSpec", "Part", "PositionEncoding",
           "StateSpec", "PreNormBlock", "TokenEmbedding", "Linear", "GatedMLP", "RMSNorm", "NoPosition",
           "RotaryPosition", "PairedRotaryPosition", "PagedAndStateSpec", "DepthAverage", "PostNormBlock", "ShortConvolution",
           "NormedTokenEmbedding", "RoutedExperts", "LatentAttention", "LatentAttentionNames", "SandwichBlock", "ParallelMixers",
           "ScaledPair", "HyperConnection", "MultiStreamBlock", "PlainMLP", "StreamReadNorm", "MatrixMemory", "MatrixMemoryNames",
           "GatedLinearAttention", "GatedLinearAttentionNames", "TimeMixing", "TimeMixingNames", "TokenShift", "ParallelGatedBlock",
           "GatedDeltaRule", "GatedDeltaNames", "DifferentialAttention", "DifferentialNames"]
