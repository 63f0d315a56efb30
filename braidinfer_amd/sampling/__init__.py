from .params import SamplingParams, uniform, uniform_key, resolve_seed
from .sampler import Sampler, SamplerState

__all__ = ["SamplingParams", "uniform", "uniform_key", "resolve_seed", "Sampler", "SamplerState"]
