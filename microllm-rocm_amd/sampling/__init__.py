from .sampler import NonFiniteLogits, Sampler, SamplingParams, uniform_for

__all__ = ["NonFiniteLogits", "Sampler", "SamplingParams", "uniform_for"]
