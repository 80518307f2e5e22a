from .params import SamplingParams
from .rng import RandomStream
from .sampler import RequestSampler, Sampler

__all__ = ["SamplingParams", "RandomStream", "RequestSampler", "Sampler"]
