from .sampler import Sampler, SamplingParams, uniform_draw

__all__ = ["Sampler", "SamplingParams", "uniform_draw"]
