from .base import Part, KvNeed, StateNeed, flat_needs
from .norm import RmsNorm, DynamicTanh
from .position import Position, NoPosition, RotaryHalfSplit, LogDistanceBias
from .mixer import Mixer, GqaAttention, GatedWindowAttention, ParallelMixers
from .memory import MatrixMemory
from .feedforward import FeedForward, GatedMlp
from .block import Block, PreNormBlock, HyperConnectionBlock
from .linear import (Matrix, linear, linear_for_sum, deferred_product, DeferredProduct, ScaledRows, WeightedDeltas,
                     StreamsWrite, as_rows, as_delta)

__all__ = ["Part", "KvNeed", "StateNeed", "flat_needs", "RmsNorm", "DynamicTanh", "Position", "NoPosition",
           "RotaryHalfSplit", "LogDistanceBias", "Mixer", "GqaAttention", "GatedWindowAttention", "ParallelMixers",
           "MatrixMemory", "FeedForward", "GatedMlp", "Block", "PreNormBlock", "HyperConnectionBlock", "linear", "Matrix",
           "WeightedDeltas"]
