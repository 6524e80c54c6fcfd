from .sampler import DeviceSampler, SamplingParams, sample_host, uniform

__all__ = ["DeviceSampler", "SamplingParams", "sample_host", "uniform"]
