from .params import SamplingParams
from .rng import uniform, request_seed
from .sampler import Sampler

__all__ = ["SamplingParams", "uniform", "request_seed", "Sampler"]
