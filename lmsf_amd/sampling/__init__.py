from .params import SAMPLING_EPS, SamplingParams
from .sampler import Sampler, SamplingRow

__all__ = ["SAMPLING_EPS", "SamplingParams", "Sampler", "SamplingRow"]
