from .base import Part, KvNeed, StateNeed
from .norm import RmsNorm
from .position import Position, NoPosition, RotaryHalfSplit
from .mixer import Mixer, GqaAttention
from .feedforward import FeedForward, GatedMlp
from .block import Block, PreNormBlock
from .linear import (Matrix, linear, linear_for_sum, deferred_product, DeferredProduct, ScaledRows,
                     as_rows, as_delta)

__all__ = ["Part", "KvNeed", "StateNeed", "RmsNorm", "Position", "NoPosition", "RotaryHalfSplit", "Mixer",
           "GqaAttention", "FeedForward", "GatedMlp", "Block", "PreNormBlock", "linear", "Matrix"]
