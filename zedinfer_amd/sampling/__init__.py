from .sampler import RequestSampler, Sampler, SamplingParams, default_sampling

__all__ = ["RequestSampler", "Sampler", "SamplingParams"]
