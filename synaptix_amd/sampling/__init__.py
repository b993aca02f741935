from .philox import Philox4x32, philox4x32_10
from .params import GenerationConfig
from .sampler import SequenceSampler, apply_filters, sample_batch

__all__ = ["Philox4x32", "philox4x32_10", "GenerationConfig", "SequenceSampler", "apply_filters", "sample_batch"]
