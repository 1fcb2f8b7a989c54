from .sampler import Sampler, SamplingParams, derive_seed, uniform_of

__all__ = ["Sampler", "SamplingParams", "derive_seed", "uniform_of"]
