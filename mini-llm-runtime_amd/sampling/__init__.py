from .sampler import NonFiniteLogits, RequestRng, Sampler, splitmix64

__all__ = ["NonFiniteLogits", "RequestRng", "Sampler", "splitmix64"]
