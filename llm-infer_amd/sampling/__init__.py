from .sampler import Sampler, request_key

__all__ = ["Sampler", "request_key"]
