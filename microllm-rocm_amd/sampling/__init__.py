from .sampler import NonFiniteLogits, Sampler, SamplingParams, Selection, uniform_for

__all__ = ["NonFiniteLogits", "Sampler", "SamplingParams", "Selection", "uniform_for"]
