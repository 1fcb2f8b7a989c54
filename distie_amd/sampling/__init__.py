from .sampler import Sampler, SamplingParams, uniform_of

__all__ = ["Sampler", "SamplingParams", "uniform_of"]
