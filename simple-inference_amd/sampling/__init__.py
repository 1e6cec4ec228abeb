from .params import SamplingParams, uniform_for, uniforms_for
from .sampler import Sampler

__all__ = ["SamplingParams", "uniform_for", "uniforms_for", "Sampler"]
