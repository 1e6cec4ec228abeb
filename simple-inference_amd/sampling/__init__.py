from .params import SamplingParams, uniform_for
from .sampler import Sampler

__all__ = ["SamplingParams", "uniform_for", "Sampler"]
