from .params import SamplingParams
from .sampler import SampleRow, Sampler, fresh_seed, uniform

__all__ = ["SamplingParams", "SampleRow", "Sampler", "fresh_seed", "uniform"]
