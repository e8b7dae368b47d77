from .sampler import Sampler, uniform_for

__all__ = ["Sampler", "uniform_for"]
