from .params import SamplingParams
from .rng import RandomStream
from .sampler import RequestSampler, Sampler, filtered_draw

__all__ = ["SamplingParams", "RandomStream", "RequestSampler", "Sampler", "filtered_draw"]
