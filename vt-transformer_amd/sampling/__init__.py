from .params import SamplingParams
from .sampler import Sampler, request_seed, uniform

__all__ = ["SamplingParams", "Sampler", "request_seed", "uniform"]
