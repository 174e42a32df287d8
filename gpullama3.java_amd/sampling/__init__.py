from .sampler import DeviceSampler, SamplingParams, sample_host, select_sampler, uniform

__all__ = ["DeviceSampler", "SamplingParams", "sample_host", "select_sampler", "uniform"]
