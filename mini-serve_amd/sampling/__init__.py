from .sampler import Sampler, SamplingArgs

__all__ = ["Sampler", "SamplingArgs"]
