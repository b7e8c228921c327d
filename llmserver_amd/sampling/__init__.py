from .sampler import Sampler, request_uniform

__all__ = ["Sampler", "request_uniform"]
