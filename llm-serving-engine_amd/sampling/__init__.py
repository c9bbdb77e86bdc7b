from .sampler import GenerationConfig, Sampler, uniform_for

__all__ = ["GenerationConfig", "Sampler", "uniform_for"]
