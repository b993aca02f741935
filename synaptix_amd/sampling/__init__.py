from .philox import Philox4x32, philox4x32_10
from .params import GenerationConfig
from .sampler import SequenceSampler, filter_batch, sample_batch

__all__ = ["Philox4x32", "philox4x32_10", "GenerationConfig", "SequenceSampler", "filter_batch", "sample_batch"]
