from .sampler import RequestSampler, Sampler, SamplingParams

__all__ = ["RequestSampler", "Sampler", "SamplingParams"]
