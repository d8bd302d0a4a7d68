from .sampler import DeviceSampler, SamplingParams, fresh_seed, sample_host, uniform
