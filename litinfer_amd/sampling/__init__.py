from .sampler import Sampler, SamplingParams, uniform

__all__ = ["Sampler", "SamplingParams", "uniform"]
