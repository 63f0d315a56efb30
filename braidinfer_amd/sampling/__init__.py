from .params import SamplingParams, uniform, resolve_seed
from .sampler import Sampler

__all__ = ["SamplingParams", "uniform", "resolve_seed", "Sampler"]
