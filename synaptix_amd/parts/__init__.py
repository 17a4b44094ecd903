from .base import Part, KvNeed, StateNeed, flat_needs
from .norm import RmsNorm, DynamicTanh
from .position import (Position, NoPosition, RotaryHalfSplit, RotaryInterleaved, LogDistanceBias, RotaryScaledHalfSplit,
                       RotaryByWavelength)
from .mixer import Mixer, GqaAttention, GatedWindowAttention, ParallelMixers, DifferentialAttention
from .memory import MatrixMemory
from .recurrent import StateSpaceMixer, ChannelDeltaMixer
from .latent import LatentAttention
from .feedforward import FeedForward, GatedMlp, RoutedExperts
from .block import Block, PreNormBlock, HyperConnectionBlock, ParallelBlock
from .linear import (Matrix, linear, linear_for_sum, deferred_product, DeferredProduct, ScaledRows, WeightedDeltas,
                     StreamsWrite, ChannelScaledDeltas, SummedDeltas, as_rows, as_delta)

__all__ = ["Part", "KvNeed", "StateNeed", "flat_needs", "RmsNorm", "DynamicTanh", "Position", "NoPosition",
           "RotaryHalfSplit", "RotaryInterleaved", "LogDistanceBias", "Mixer", "GqaAttention", "GatedWindowAttention", "ParallelMixers",
           "MatrixMemory", "LatentAttention", "FeedForward", "GatedMlp", "RoutedExperts", "Block", "PreNormBlock",
           "HyperConnectionBlock", "ParallelBlock", "linear", "Matrix", "WeightedDeltas", "ChannelScaledDeltas", "SummedDeltas", "RotaryScaledHalfSplit",
           "DifferentialAttention", "StateSpaceMixer", "ChannelDeltaMixer", "RotaryByWavelength"]
