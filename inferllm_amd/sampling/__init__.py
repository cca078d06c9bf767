from .params import SamplingParams, request_seed, splitmix64, uniform
from .sampler import Sampler

__all__ = ["SamplingParams", "Sampler", "request_seed", "splitmix64", "uniform"]
