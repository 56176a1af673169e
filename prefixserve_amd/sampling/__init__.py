from .sampler import Sampler, request_key, uniform_for

__all__ = ["Sampler", "request_key", "uniform_for"]
